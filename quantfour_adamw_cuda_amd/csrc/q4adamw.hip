// Fused 4-bit AdamW step for MI355X (gfx950): kernels, launchers and the C ABI
// declared in include/q4adamw.h.
//
// Build: hipcc --offload-arch=gfx950 -O3 -ffp-contract=off -shared -fPIC
// (-ffp-contract=off matters: the moment updates must be individually rounded
// fp32 multiplies and adds; fused multiply-adds appear only where written out).
//
// Work decomposition of the fused kernel (shaped by measurement: HBM on this part
// streams best when every wave is short-lived, touches 1 KiB of the widest stream
// with ONE 16-byte access per lane, and every access is marked non-temporal)
//   tile    = one wave64, one pass; a lane owns 16 bytes of the parameter stream:
//             4 consecutive fp32 parameters (tile = 256 elements = 2 quantization
//             blocks, a block = 32 lanes, abs-max by one v_permlane16_swap plus four
//             DPP row steps) or 8 consecutive bf16 parameters (tile = 512 elements =
//             4 blocks, a block = one 16-lane DPP row).  No LDS traffic and no
//             barrier in the reduction.
//   chunk   = 4 tiles of ONE tensor = one 256-thread workgroup.
//   launch  = all chunks of up to kMaxTensors tensors.  The tensor descriptors and
//             the per-tensor first-chunk prefix travel in the kernel arguments, so
//             a workgroup finds its tensor with two scalar loads from the kernarg
//             segment and nothing is staged in device memory.  Workgroup ids are
//             dealt round-robin to the 8 XCDs; the kernel maps id -> chunk so that
//             each XCD walks one contiguous eighth of the chunk space, which keeps
//             neighbouring blocks' scales (4 bytes per block) in one L2.
// Per element the kernel reads p, g and one nibble of each moment, and writes p
// and one nibble of each moment; per block it reads and writes two fp32 scales.
#include <hip/hip_runtime.h>
#include <float.h>
#include <math.h>
#include <stdint.h>
#include <string.h>

#include <string>

#include "../../include/q4adamw.h"
#include "q4adamw_tables.h"

namespace q4 {

constexpr int kWaves = 4;                  // waves per workgroup
constexpr int kThreads = kWaves * 64;
constexpr int kMaxTensors = 48;            // tensors per fused launch
constexpr int kSmallChunk = 1024;          // elements per workgroup, non-quantized kernel
constexpr int kMaxSmallTensors = 80;

// derived on the host exactly as optim/cuda_adamw_kernels.cu:435-440
struct StepConsts {
  float b1, b2, r1, r2;  // beta1, beta2, 1-beta1, 1-beta2
  float wdu, ss;         // 1 - lr*wd, lr / (1 - beta1^t)
  float c2s;             // sqrt(1 - beta2^t)
  float eps;
  // the fused kernel's parameter update p*wdu - m'/(sqrt(v')*den_scale + den_eps), the
  // step size folded into the denominator: 1/(c2s*ss) and eps/ss
  float den_scale, den_eps;
};

// What a launch does to the gradients besides reading them (kernels with EXT only).
struct GradOps {
  float scale;             // host part of the multiplier
  uint32_t zero;           // non-zero: overwrite the gradients with zeros once they are read
  const float *scale_dev;  // device part of the multiplier, or null
  const float *skip;       // device flag, or null: non-zero turns the launch into a no-op
};

struct TensorDesc {  // 56 bytes
  void *p;
  const void *g;
  uint8_t *m;
  uint8_t *v;
  float *sm;
  float *sv;
  int64_t numel;
};

// Kernel arguments of one fused launch (about 3 KiB, passed by value).
// first_chunk[i] = index of tensor i's first chunk; entries past ntensors hold
// 0x7fffffff (more than any chunk index).  pivot[k] = first_chunk[8k] lets a workgroup find its tensor with two
// wide scalar loads.
struct FusedArgs {
  static constexpr int kCapacity = kMaxTensors;
  static constexpr int kPivots = (kMaxTensors + 7) / 8;
  StepConsts sc;
  GradOps go;
  int ntensors;
  uint32_t nchunks;        // chunks in this launch
  uint32_t chunks_per_xcd; // ceil(nchunks / 8); the grid has 8 * chunks_per_xcd workgroups
  uint32_t pivot[kPivots];
  uint32_t first_chunk[kPivots * 8];
  TensorDesc desc[kMaxTensors];
  uint32_t sr_salt[kMaxTensors];  // stochastic rounding: the tensors' noise salts of this step
};

struct SmallDesc {  // 40 bytes
  void *p;
  const void *g;
  float *m;
  float *v;
  int64_t numel;
};

struct SmallArgs {
  static constexpr int kCapacity = kMaxSmallTensors;
  static constexpr int kPivots = (kMaxSmallTensors + 7) / 8;
  StepConsts sc;
  GradOps go;
  int ntensors;
  uint32_t pivot[kPivots];
  uint32_t first_chunk[kPivots * 8];
  SmallDesc desc[kMaxSmallTensors];
};

// One tensor whose second moment is rank-1 scaled (a rows x cols matrix, row-major).
struct Rank1Desc {  // 104 bytes
  void *p;
  const void *g;
  uint8_t *m;
  uint8_t *v;
  float *sm;          // block scales of the first moment
  float *rmax;        // current statistics of the second moment: rows, cols floats
  float *cmax;
  float *rmax_next;   // the step's new statistics (all zero between steps)
  float *cmax_next;
  int64_t numel;      // rows * cols
  int64_t rows;
  int64_t cols;
  // division of a 32-bit number by cols / 8 as multiply-high, add and shifts
  // (round-up method: exact for every 32-bit dividend)
  uint32_t div_magic;
  uint32_t div_shift;
};

struct FastDiv {
  uint32_t magic, shift;
};

// n / d for the divisor the pair was made for
__host__ __device__ __forceinline__ uint32_t fast_div(uint32_t n, uint32_t magic, uint32_t shift) {
#if defined(__HIP_DEVICE_COMPILE__)
  const uint32_t t = __umulhi(n, magic);
#else
  const uint32_t t = (uint32_t)(((uint64_t)n * magic) >> 32);
#endif
  return (t + ((n - t) >> 1)) >> shift;
}

static FastDiv make_fast_div(uint32_t d) {  // d >= 2
  uint32_t l = 0;
  while ((1ull << l) < d) ++l;                     // ceil(log2 d) >= 1
  FastDiv f;
  f.magic = (uint32_t)((((1ull << l) - d) << 32) / d + 1);
  f.shift = l - 1;
  return f;
}

constexpr int kMaxRank1Tensors = 32;

// Kernel arguments of the rank-1 launches.  The update kernel indexes chunks of
// kChunk flat elements like FusedArgs; the statistics kernel indexes tiles of
// kStatRows rows x kStatCols columns (stat_first_chunk, stat_col_groups).
struct Rank1Args {
  static constexpr int kCapacity = kMaxRank1Tensors;
  static constexpr int kPivots = (kMaxRank1Tensors + 7) / 8;
  StepConsts sc;
  GradOps go;
  int ntensors;
  uint32_t nchunks;
  uint32_t chunks_per_xcd;
  uint32_t pivot[kPivots];
  uint32_t first_chunk[kPivots * 8];
  Rank1Desc desc[kMaxRank1Tensors];
};

struct Rank1StatArgs {
  static constexpr int kCapacity = kMaxRank1Tensors;
  static constexpr int kPivots = (kMaxRank1Tensors + 7) / 8;
  float b2, r2;
  GradOps go;
  int ntensors;
  uint32_t nchunks;
  uint32_t pivot[kPivots];
  uint32_t first_chunk[kPivots * 8];
  uint32_t col_groups[kMaxRank1Tensors];   // column groups per row group of tensor t
  struct Desc {
    const void *g;
    const uint8_t *v;
    const float *rmax;
    const float *cmax;
    float *rmax_next;
    float *cmax_next;
    int64_t rows;
    int64_t cols;
  } desc[kMaxRank1Tensors];
};

// Gradient-norm launch: every workgroup walks chunks of 32 KiB with a grid stride.
constexpr int kMaxNormTensors = 160;
constexpr int kNormPartials = Q4ADAMW_NORM_WORKSPACE_BYTES / 8;  // workgroups = fp64 partial sums
constexpr int kNormChunkBytes = 32768;                          // 8 16-byte loads per thread

struct NormDesc {
  const void *g;
  int64_t numel;
};

struct NormArgs {
  static constexpr int kCapacity = kMaxNormTensors;
  static constexpr int kPivots = (kMaxNormTensors + 7) / 8;
  double *partials;   // kNormPartials sums, one per workgroup
  uint32_t nchunks;
  uint32_t first;     // non-zero: the partial sums are overwritten, otherwise added to
  int ntensors;
  uint32_t pivot[kPivots];
  uint32_t first_chunk[kPivots * 8];
  NormDesc desc[kMaxNormTensors];
};

static_assert(sizeof(FusedArgs) <= 4096 && sizeof(SmallArgs) <= 4096 && sizeof(NormArgs) <= 4096 &&
                  sizeof(Rank1Args) <= 4096 && sizeof(Rank1StatArgs) <= 4096,
              "kernel arguments are limited to 4 KiB");

// the first-moment bucket table (see q4adamw_tables.h), copied into LDS by every
// workgroup at start-up, one entry per thread
__device__ const HalfTable kHalfTable = make_half_table();
// stochastic rounding: code-book entries per bucket and the 17 intervals between them
__device__ const SrHalfTable kSrHalfTable = make_sr_half_table();
__device__ const SrIntervalTable kSrIntervals = make_sr_interval_table();
// first-moment code book for kernels that index it per lane
__device__ const uint32_t kQmapMDev[16] = {
    0xbf633333u, 0xbf29999au, 0xbee00000u, 0xbe59999au, 0xbd9eb852u, 0xbd051eb8u,
    0xbbb43958u, 0x00000000u, 0x3bb43958u, 0x3d051eb8u, 0x3d9eb852u, 0x3e59999au,
    0x3ee00000u, 0x3f29999au, 0x3f633333u, 0x3f800000u};

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

// Full tiles go through buffer instructions: the tile's base address sits in a
// scalar resource descriptor and each lane supplies a 32-bit byte offset, so no
// vector ALU work goes into addresses.  Cache policy of the streamed tensors: the
// non-temporal hint (bit 1) plus system scope (sc1, bit 4); every datum is touched
// once, and with the wider scope the streams measure 1.5 % faster than with the hint
// alone (and 11 % faster than without either).
typedef __amdgpu_buffer_rsrc_t rsrc_t;
constexpr int kNt = 2 | 16;
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

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return bits2f(h << 16); }

__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {  // round to nearest even
  return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)f);
}

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

// two fp32 -> two bf16 (round to nearest even) in one 32-bit word, lo in the low half
__device__ __forceinline__ uint32_t pack_bf16_pair(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, bf16x2));
}

__device__ __forceinline__ void widen_bf16_pair(uint32_t w, float &lo, float &hi) {
  lo = bits2f(w << 16);
  hi = bits2f(w & 0xffff0000u);
}

// N consecutive elements (N = 4 or 8) starting at element e0 of the tile at base
template <bool BF, int N, bool FULL>
__device__ __forceinline__ void load_elems(const void *base, uint32_t e0, int nv, float (&x)[N]) {
  if (FULL) {
    if (BF && N == 4) {
      const u32x2 w = __builtin_amdgcn_raw_buffer_load_b64(tile_rsrc(base), e0 * 2, 0, kNt);
      widen_bf16_pair(w.x, x[0], x[1]);
      widen_bf16_pair(w.y, x[2], x[3]);
    } else if (BF) {
      const u32x4 w = __builtin_amdgcn_raw_buffer_load_b128(tile_rsrc(base), e0 * 2, 0, kNt);
      widen_bf16_pair(w.x, x[0], x[1]);
      widen_bf16_pair(w.y, x[2], x[3]);
      widen_bf16_pair(w.z, x[N - 4], x[N - 3]);
      widen_bf16_pair(w.w, x[N - 2], x[N - 1]);
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
        x[j] = BF ? bf16_bits_to_f32(as_global<const uint16_t>(base)[e0 + j])
                  : as_global<const float>(base)[e0 + j];
      }
    }
  }
}

template <bool BF, int N, bool FULL>
__device__ __forceinline__ void store_elems(void *base, uint32_t e0, int nv, const float (&x)[N]) {
  if (FULL) {
    if (BF && N == 4) {
      u32x2 w;
      w.x = pack_bf16_pair(x[0], x[1]);
      w.y = pack_bf16_pair(x[2], x[3]);
      __builtin_amdgcn_raw_buffer_store_b64(w, tile_rsrc(base), e0 * 2, 0, kNt);
    } else if (BF) {
      u32x4 w;
      w.x = pack_bf16_pair(x[0], x[1]);
      w.y = pack_bf16_pair(x[2], x[3]);
      w.z = pack_bf16_pair(x[N - 4], x[N - 3]);
      w.w = pack_bf16_pair(x[N - 2], x[N - 1]);
      __builtin_amdgcn_raw_buffer_store_b128(w, tile_rsrc(base), e0 * 2, 0, kNt);
    } else {
#pragma unroll
      for (int k = 0; k < N; k += 4) {
        const u32x4 w = {f2bits(x[k]), f2bits(x[k + 1]), f2bits(x[k + 2]), f2bits(x[k + 3])};
        __builtin_amdgcn_raw_buffer_store_b128(w, tile_rsrc(base), (e0 + k) * 4, 0, kNt);
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < N; ++j) {
      if (j < nv) {
        if (BF) as_global<uint16_t>(base)[e0 + j] = (uint16_t)f32_to_bf16_bits(x[j]);
        else as_global<float>(base)[e0 + j] = x[j];
      }
    }
  }
}

// zeros over the N elements that load_elems<BF, N, FULL> read
template <bool BF, int N, bool FULL>
__device__ __forceinline__ void zero_elems(void *base, uint32_t e0, int nv) {
  if (FULL) {
    const u32x4 z4 = {0u, 0u, 0u, 0u};
    if (BF && N == 4) {
      const u32x2 z2 = {0u, 0u};
      __builtin_amdgcn_raw_buffer_store_b64(z2, tile_rsrc(base), e0 * 2, 0, kNt);
    } else if (BF) {
      __builtin_amdgcn_raw_buffer_store_b128(z4, tile_rsrc(base), e0 * 2, 0, kNt);
    } else {
#pragma unroll
      for (int k = 0; k < N; k += 4)
        __builtin_amdgcn_raw_buffer_store_b128(z4, tile_rsrc(base), (e0 + k) * 4, 0, kNt);
    }
  } else {
#pragma unroll
    for (int j = 0; j < N; ++j) {
      if (j < nv) {
        if (BF) as_global<uint16_t>(base)[e0 + j] = 0;
        else as_global<float>(base)[e0 + j] = 0.0f;
      }
    }
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

// A 32-bit integer mixer (two multiply-xorshift rounds) for the rounding noise.
__host__ __device__ __forceinline__ uint32_t lowbias32(uint32_t x) {
  x ^= x >> 16;
  x *= 0x7FEB352Du;
  x ^= x >> 15;
  x *= 0x846CA68Bu;
  x ^= x >> 16;
  return x;
}

// noise in (0, 1) from a 16-bit number: (2 n + 1) / 2^17, exact
__device__ __forceinline__ float sr_noise_value(uint32_t n16) {
  return __builtin_fmaf((float)n16, 1.52587890625e-05f, 7.62939453125e-06f);
}

// Stochastic rounding, exact form (the closed form of quantize_bsearch<STOCHASTIC>,
// optim/adamw_fourbit_triton.py:1050-1075, without its division): IEEE quotient, its
// interval [Q[k], Q[k+1]) among the code-book entries, upper code iff
// noise * (Q[k+1] - Q[k]) < q - Q[k].  0/0 is NaN and gets code 0.
template <bool SECOND, int N>
__device__ __forceinline__ uint32_t quantize_exact_sr(const Vals<N> &v, float scale, const Vals<N> &noise) {
  uint32_t word = 0;
#pragma unroll
  for (int j = 0; j < N; ++j) {
    const float q = v.x[j] / scale;
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
    const bool up = noise.x[j] * width < q - lower;
    int c = (int)k_raw - 1 + (up ? 1 : 0);
    c = c < 0 ? 0 : (c > 15 ? 15 : c);
    word |= (uint32_t)c << (4 * j);
  }
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

// Byte BYTE of x, times 8 (the byte offset of an 8-byte table entry), as one SDWA
// shift; `three` is the shift amount in a register.
template <int BYTE>
__device__ __forceinline__ uint32_t byte_times8(uint32_t x, uint32_t three) {
  static_assert(BYTE >= 0 && BYTE <= 3, "");
  uint32_t r;
#define Q4_SDWA_SHIFT(SEL)                                                                          \
  asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:" SEL \
      : "=v"(r) : "v"(three), "v"(x))
  if (BYTE == 0) Q4_SDWA_SHIFT("BYTE_0");
  else if (BYTE == 1) Q4_SDWA_SHIFT("BYTE_1");
  else if (BYTE == 2) Q4_SDWA_SHIFT("BYTE_2");
  else Q4_SDWA_SHIFT("BYTE_3");
#undef Q4_SDWA_SHIFT
  return r;
}

// byte_times8 with the byte chosen by a loop index of an unrolled loop
__device__ __forceinline__ uint32_t entry_offset(uint32_t x, int byte, uint32_t three) {
  switch (byte) {
    case 0: return byte_times8<0>(x, three);
    case 1: return byte_times8<1>(x, three);
    case 2: return byte_times8<2>(x, three);
    default: return byte_times8<3>(x, three);
  }
}

// 1/s to within half an ulp for s in [2^-100, 2^100]: hardware estimate plus one
// Newton step
__device__ __forceinline__ float refined_rcp(float s) {
  const float r0 = __builtin_amdgcn_rcpf(s);
  const float e = __builtin_fmaf(-s, r0, 1.0f);
  return __builtin_fmaf(e, r0, r0);
}

constexpr float kScaleLo = 7.888609052210118e-31f;   // 2^-100
constexpr float kScaleHi = 1.2676506002282294e+30f;  // 2^100
constexpr float kVGuard = 7.62939453125e-06f;        // 2^-17, in units of 16*q

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
//   [0, 256)    the waves' private dequantization tables: per wave 64 entries, per
//               quantization block 16 entries {code_book_m[i] * scale_m,
//               code_book_v[i] * scale_v}, so that dequantizing an element is one read
//               and an entry number fits a byte
//   [256, 512)  bucket table of the first-moment quantizer, indexed by the high byte
//               of the quotient as a half
//   [512, 529)  stochastic rounding only: the first moment's interval table
constexpr uint32_t kLdsBuckets = 64 * kWaves;
constexpr uint32_t kLdsIntervals = kLdsBuckets + kHalfTableEntries;
constexpr uint32_t kLdsEntries = kLdsIntervals + 32;
static_assert(kLdsBuckets == 256, "dequantization entry numbers must fit a byte");
static_assert(kThreads == (int)kHalfTableEntries, "one bucket table entry per thread");

// What a thread fetches from the constant tables as the very first thing it does.
struct TableSlot {
  uint2 entry;     // bucket table entry number tid
  float qm;        // first-moment code-book value number (lane & 15)
  uint2 interval;  // stochastic rounding: interval table entry number tid (tid < 17)
};

template <bool SR>
__device__ __forceinline__ TableSlot request_table_slot(int tid) {
  TableSlot s;
  if (SR) {
    const SrEntry e = kSrHalfTable.e[tid];
    s.entry = make_uint2(e.thr, e.base);
    const SrInterval iv = kSrIntervals.e[tid < 17 ? tid : 0];
    s.interval = make_uint2(f2bits(iv.lower), f2bits(iv.width));
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

// Geometry of the fused kernel: a lane owns 16 bytes of the widest of the parameter and
// gradient streams, so that no stream needs two accesses per lane.
template <bool PBF, bool GBF>
struct Geometry {
  static constexpr int kEpl = (PBF && GBF) ? 8 : 4;      // elements per lane
  static constexpr int kTile = 64 * kEpl;                // elements per wave
  static constexpr int kChunk = kTile * kWaves;          // elements per workgroup
  static constexpr int kLanesPerBlock = Q4ADAMW_BLOCK / kEpl;   // 32 or 16
  static constexpr int kBlocksPerTile = kTile / Q4ADAMW_BLOCK;  // 2 or 4
};

// ---------------------------------------------------------------------------
// one tile (256 or 512 elements) of one tensor
// ---------------------------------------------------------------------------
// EXT: gradients are multiplied by gscale (one rounded fp32 multiplication per
// element, before anything else uses them) and, if zero_g, overwritten with zeros.
// RANK1 (Desc = Rank1Desc): the second moment's scale is min(row maximum, column
// maximum) per element instead of one value per block: old statistics dequantize, the
// step's new statistics (complete before this kernel starts) quantize.
// SR: both moments are rounded stochastically between the two neighbouring code-book
// entries; the noise of element e is a hash of e and the tensor's salt of this step.
template <bool PBF, bool GBF, bool FULL, bool EXT, bool RANK1, bool SR, typename Desc>
__device__ __forceinline__ void process_tile(const Desc &T, int64_t tile, int lane, int wave, int tid,
                                             const StepConsts &sc, uint2 *lds, const TableSlot &slot,
                                             float gscale, bool zero_g, uint32_t salt) {
  static_assert(!(SR && RANK1), "stochastic rounding is built for block scaling only");
  using G = Geometry<PBF, GBF>;
  constexpr int N = G::kEpl;
  // Uniform (scalar) part of every address: the tile's first element, byte and
  // block; the per-lane part is a small 32-bit offset.
  const int64_t numel = T.numel;
  const int64_t tb = tile * G::kTile;
  const void *p_tile = static_cast<const char *>(T.p) + tb * (PBF ? 2 : 4);
  const void *g_tile = static_cast<const char *>(T.g) + tb * (GBF ? 2 : 4);
  const uint8_t *m_tile = T.m + (tb >> 1);
  const uint8_t *v_tile = T.v + (tb >> 1);
  const float *sm_tile = T.sm + tile * G::kBlocksPerTile;
  const float *sv_tile = nullptr;
  if constexpr (!RANK1) sv_tile = T.sv + tile * G::kBlocksPerTile;
  const uint32_t e0 = (uint32_t)lane * N;                          // first element of this lane in the tile
  const uint32_t blk = (uint32_t)lane / G::kLanesPerBlock;         // which of the tile's blocks
  const uint32_t code_off = (uint32_t)lane * (N / 2);              // byte offset of this lane's codes
  int nv = N;
  bool blk_ok = true;
  if (!FULL) {
    const int64_t rem = numel - tb - (int64_t)e0;
    nv = rem >= N ? N : (rem > 0 ? (int)rem : 0);
    blk_ok = tb + (int64_t)blk * Q4ADAMW_BLOCK < numel;
  }

  // rank-1: this lane's row maxima (old, new) and its N column maxima (old, new)
  float r_old = 0.0f, r_new = 0.0f;
  Vals<N> c_old, c_new;
  if constexpr (RANK1) {
    // (row, column) of the tile's first element, in units of 8 elements so that the
    // division is a 32-bit one.  A tile is shorter than a row, so a lane is in that
    // row or in the next one.
    const uint32_t tb8 = (uint32_t)(tb >> 3), cols8 = (uint32_t)(T.cols >> 3);  // numel < 2^35
    const uint32_t row32 = fast_div(tb8, T.div_magic, T.div_shift);
    const int64_t row = row32;
    const uint32_t col0 = (tb8 - row32 * cols8) << 3;
    uint32_t col = col0 + e0;
    const bool wrapped = col >= (uint32_t)T.cols;
    if (wrapped) col -= (uint32_t)T.cols;
    const int64_t last = T.rows - 1;
    const int64_t ra = row < last ? row : last, rb = row + 1 < last ? row + 1 : last;  // past-the-end lanes stay in bounds
    const float r_old_a = as_global<const float>(T.rmax)[ra], r_old_b = as_global<const float>(T.rmax)[rb];
    const float r_new_a = as_global<const float>(T.rmax_next)[ra], r_new_b = as_global<const float>(T.rmax_next)[rb];
    r_old = wrapped ? r_old_b : r_old_a;
    r_new = wrapped ? r_new_b : r_new_a;
#pragma unroll
    for (int k = 0; k < N; k += 4) {
      const u32x4 a = __builtin_amdgcn_raw_buffer_load_b128(tile_rsrc(T.cmax), (col + k) * 4u, 0, 0);
      const u32x4 b = __builtin_amdgcn_raw_buffer_load_b128(tile_rsrc(T.cmax_next), (col + k) * 4u, 0, 0);
      c_old.x[k] = bits2f(a.x); c_old.x[k + 1] = bits2f(a.y); c_old.x[k + 2] = bits2f(a.z); c_old.x[k + 3] = bits2f(a.w);
      c_new.x[k] = bits2f(b.x); c_new.x[k + 1] = bits2f(b.y); c_new.x[k + 2] = bits2f(b.z); c_new.x[k + 3] = bits2f(b.w);
    }
  }

  float p[N], g[N];
  load_elems<PBF, N, FULL>(p_tile, e0, nv, p);
  load_elems<GBF, N, FULL>(g_tile, e0, nv, g);
  if (EXT) {
#pragma unroll
    for (int j = 0; j < N; ++j) g[j] *= gscale;
    if (zero_g) zero_elems<GBF, N, FULL>(const_cast<void *>(g_tile), e0, nv);
  }
  uint32_t mw = 0, vw = 0;
  if (FULL) {
    if (N == 4) {
      mw = __builtin_amdgcn_raw_buffer_load_b16(tile_rsrc(m_tile), code_off, 0, kNt);
      vw = __builtin_amdgcn_raw_buffer_load_b16(tile_rsrc(v_tile), code_off, 0, kNt);
    } else {
      mw = __builtin_amdgcn_raw_buffer_load_b32(tile_rsrc(m_tile), code_off, 0, kNt);
      vw = __builtin_amdgcn_raw_buffer_load_b32(tile_rsrc(v_tile), code_off, 0, kNt);
    }
  } else {
    const gptr<const uint8_t> mb = as_global<const uint8_t>(m_tile) + code_off;
    const gptr<const uint8_t> vb = as_global<const uint8_t>(v_tile) + code_off;
    const int nb = (nv + 1) >> 1;
#pragma unroll
    for (int k = 0; k < N / 2; ++k) {
      if (k < nb) {
        mw |= (uint32_t)mb[k] << (8 * k);
        vw |= (uint32_t)vb[k] << (8 * k);
      }
    }
  }
  float sm_old = 0.0f, sv_old = 0.0f;
  if (FULL) {
    // scales are 4 bytes per block: cached, so that neighbouring blocks share lines
    sm_old = bits2f(__builtin_amdgcn_raw_buffer_load_b32(tile_rsrc(sm_tile), blk * 4u, 0, 0));
    if (!RANK1) sv_old = bits2f(__builtin_amdgcn_raw_buffer_load_b32(tile_rsrc(sv_tile), blk * 4u, 0, 0));
  } else if (blk_ok) {
    sm_old = as_global<const float>(sm_tile)[blk];
    if (!RANK1) sv_old = as_global<const float>(sv_tile)[blk];
  }
  if (RANK1) sv_old = 1.0f;  // the table holds the bare code book; the scale follows per element
  // this block's dequantization table: entry i = {code_book_m[i] * scale_m,
  // code_book_v[i] * scale_v} (cuda_adamw_kernels.cu:340,343), written by the block's
  // lanes (lane & 15 = i) into the wave's private LDS region
  char *lds_bytes = reinterpret_cast<char *>(lds);
  const uint32_t cb_entry = (uint32_t)wave * 64u + blk * 16u;  // entry number of code 0
  *reinterpret_cast<float2 *>(lds_bytes + (cb_entry + ((uint32_t)lane & 15u)) * 8u) =
      make_float2(slot.qm * sm_old, qmap_v(lane & 15) * sv_old);
  setup_tables<SR>(lds, tid, slot);

  // entry numbers of the lane's codes, one per byte: even elements, odd elements
  const uint32_t three = 3u;
  const uint32_t cb_bytes = cb_entry * 0x01010101u;
  const uint32_t m_even = and_or(mw, 0x0F0F0F0Fu, cb_bytes), m_odd = and_or(mw >> 4, 0x0F0F0F0Fu, cb_bytes);
  const uint32_t v_even = and_or(vw, 0x0F0F0F0Fu, cb_bytes), v_odd = and_or(vw >> 4, 0x0F0F0F0Fu, cb_bytes);

  // dequantize, update moments and parameter (cuda_adamw_kernels.cu:334-351)
  Vals<N> mn, vn;
  float am = 0.0f, av = 0.0f;
#pragma unroll
  for (int j = 0; j < N; ++j) {
    const uint32_t mo = entry_offset(j & 1 ? m_odd : m_even, j >> 1, three);
    const uint32_t vo = entry_offset(j & 1 ? v_odd : v_even, j >> 1, three);
    const float m_old = *reinterpret_cast<const float *>(lds_bytes + mo);
    float v_old = *reinterpret_cast<const float *>(lds_bytes + vo + 4);
    if constexpr (RANK1) v_old *= __builtin_fminf(r_old, c_old.x[j]);  // adamw_fourbit_triton.py:520-527
    const float gj = g[j];
    float m = sc.b1 * m_old + sc.r1 * gj;
    float v = sc.b2 * v_old + sc.r2 * (gj * gj);
    if (!FULL && j >= nv) { m = 0.0f; v = 0.0f; }
    // parameter: only this part may use the hardware's 1-ulp sqrt and reciprocal
    const float den = __builtin_fmaf(__builtin_amdgcn_sqrtf(v), sc.den_scale, sc.den_eps);
    p[j] = __builtin_fmaf(-m, __builtin_amdgcn_rcpf(den), p[j] * sc.wdu);
    mn.x[j] = m;
    vn.x[j] = v;
    am = __builtin_fmaxf(am, __builtin_fabsf(m));
    av = __builtin_fmaxf(av, v);
  }
  store_elems<PBF, N, FULL>(const_cast<void *>(p_tile), e0, nv, p);

  // block scales (exact: max is order independent)
  const float v_lane_max = av;
  if (G::kLanesPerBlock == 32) {
    block_max32_pair(am, av);
  } else {
    am = row_max16(am);
    if (!RANK1) av = row_max16(av);
  }
  if (blk_ok && (lane & (G::kLanesPerBlock - 1)) == 0) {
    if (FULL) {
      __builtin_amdgcn_raw_buffer_store_b32(f2bits(am), tile_rsrc(sm_tile), blk * 4u, 0, 0);
      if (!RANK1) __builtin_amdgcn_raw_buffer_store_b32(f2bits(av), tile_rsrc(sv_tile), blk * 4u, 0, 0);
    } else {
      as_global<float>(sm_tile)[blk] = am;
      if (!RANK1) as_global<float>(sv_tile)[blk] = av;
    }
  }

  // fast quantization: multiply by a refined reciprocal, decide every code whose
  // quotient is clear of all thresholds, flag the rest
  const bool safe_m = am >= kScaleLo && am <= kScaleHi;
  const bool safe_v = RANK1 || (av >= kScaleLo && av <= kScaleHi);
  const float rm = safe_m ? refined_rcp(am) : 0.0f;
  const float rv16 = (safe_v && !RANK1) ? refined_rcp(av) * 16.0f : 0.0f;  // exact scaling
  bool redo = (!safe_m && am != 0.0f) || (!safe_v && av != 0.0f);
  float vfrac = 1.0f;  // smallest distance of a scaled second moment above a threshold
  // rank-1: the new scale of every element and 16 / scale.  The hardware reciprocal's
  // one ulp is well inside the second moment's guard band (2^-17 in units of 16 q), so
  // it goes unrefined.  Scales below the safe range are clamped for the reciprocal: a
  // zero value under a zero scale then still gets code 0; any other value under such a
  // scale sends the lane to the exact path.
  Vals<N> s_new, inv16;
  if constexpr (RANK1) {
    float c_min = c_new.x[0];
#pragma unroll
    for (int j = 0; j < N; ++j) {
      const float sj = __builtin_fminf(r_new, c_new.x[j]);   // adamw_fourbit_triton.py:749-755
      s_new.x[j] = sj;
      c_min = __builtin_fminf(c_min, c_new.x[j]);
      inv16.x[j] = __builtin_amdgcn_rcpf(__builtin_fmaxf(sj, kScaleLo)) * 16.0f;
    }
    // every scale is at most r_new and at least min(r_new, c_min)
    redo |= r_new > kScaleHi || (__builtin_fminf(r_new, c_min) < kScaleLo && v_lane_max != 0.0f);
  }
  uint32_t mword = 0, vword = 0;
  Vals<N> um, uv;  // stochastic rounding: the elements' noise
  if constexpr (SR) {
    // key = low half of the element index, xor the salt, xor the mixed high half
    const uint32_t tile_salt = salt ^ ((uint32_t)((uint64_t)tb >> 32) * 0x9E3779B9u);
    const uint32_t first = (uint32_t)tb + e0;   // a tile never straddles a multiple of 2^32
#pragma unroll
    for (int j = 0; j < N; ++j) {
      const uint32_t h = lowbias32((first + (uint32_t)j) ^ tile_salt);
      um.x[j] = sr_noise_value(h >> 16);
      uv.x[j] = sr_noise_value(h & 0xffffu);
    }
  }
#pragma unroll
  for (int j = 0; j < N; j += 2) {
    // first moment: the quotients' bucket entries, two quotients per conversion
    const float q0 = mn.x[j] * rm, q1 = mn.x[j + 1] * rm;
    const uint32_t halves = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(q0, q1));
    const uint2 ent0 = *reinterpret_cast<const uint2 *>(lds_bytes + kLdsBuckets * 8u + byte_times8<1>(halves, three));
    const uint2 ent1 = *reinterpret_cast<const uint2 *>(lds_bytes + kLdsBuckets * 8u + byte_times8<3>(halves, three));
    if constexpr (SR) {
      // interval among the code-book entries, then up iff noise * width < q - lower end;
      // a comparison closer than the quotient's error goes to the exact path
      const float qq[2] = {q0, q1};
      const uint2 ent[2] = {ent0, ent1};
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const uint32_t k_raw = ent[h].y + (qq[h] >= bits2f(ent[h].x) ? 1u : 0u);
        const uint2 iv = *reinterpret_cast<const uint2 *>(lds_bytes + kLdsIntervals * 8u + k_raw * 8u);
        const float d = qq[h] - bits2f(iv.x), t = um.x[j + h] * bits2f(iv.y);
        redo |= __builtin_fabsf(t - d) <= __builtin_fabsf(qq[h]) * 4.76837158203125e-07f;  // 2^-21: 4 ulps
        mword = __builtin_amdgcn_alignbit(k_raw - 1u + (t < d ? 1u : 0u), mword, 4);
      }
    } else {
      const bool hi0 = q0 > bits2f(ent0.y), hi1 = q1 > bits2f(ent1.y);
      redo |= (hi0 != (q0 > bits2f(ent0.x))) | (hi1 != (q1 > bits2f(ent1.x)));
      // base code in the entry's low nibble, plus one above the threshold; every
      // code enters the word at the top and moves down four bits per later element
      mword = __builtin_amdgcn_alignbit(ent0.x + (hi0 ? 1u : 0u), mword, 4);
      mword = __builtin_amdgcn_alignbit(ent1.x + (hi1 ? 1u : 0u), mword, 4);
    }

    // second moment: thresholds at 16q = k + 0.5, k = 1..15
#pragma unroll
    for (int k = j; k < j + 2; ++k) {
      if constexpr (SR) {
        // code-book entries at 16 q = 1..16: interval number floor(16 q), position in
        // it fract(16 q), up iff noise < position; the ends clamp
        const float q16 = vn.x[k] * rv16;
        const float kf = __builtin_floorf(q16), d16 = q16 - kf;
        redo |= __builtin_fabsf(uv.x[k] - d16) <= kVGuard;
        const float cf = __builtin_amdgcn_fmed3f(kf + (uv.x[k] < d16 ? 0.0f : -1.0f), 0.0f, 15.0f);
        vword = __builtin_amdgcn_alignbit((uint32_t)(int)cf, vword, 4);
      } else {
        const float t = __builtin_fmaf(vn.x[k], RANK1 ? inv16.x[k] : rv16, kVGuard - 0.5f);
        vfrac = __builtin_fminf(vfrac, __builtin_amdgcn_fractf(t));
        // t > -1, so truncation gives 0 for t < 0
        vword = __builtin_amdgcn_alignbit((uint32_t)(int)t, vword, 4);
      }
    }
  }
  if (N == 4) {
    mword >>= 16;
    vword >>= 16;
  }
  redo |= vfrac < 2.0f * kVGuard;
  if (__builtin_expect(redo, 0)) {
    if constexpr (SR) {
      mword = quantize_exact_sr<false, N>(mn, am, um);
      vword = quantize_exact_sr<true, N>(vn, av, uv);
    } else {
      mword = quantize_exact<false, N>(mn, am);
      if constexpr (RANK1) vword = quantize_exact_scales<N>(vn, s_new);
      else vword = quantize_exact<true, N>(vn, av);
    }
  }
  if (am == 0.0f) mword = 0;  // 0/0: code 0 for the whole block
  if (!FULL) {
    const uint32_t keep = nv >= 8 ? 0xffffffffu : ((1u << (4 * nv)) - 1u);
    mword &= keep;
    vword &= keep;
  }

  if (FULL) {
    if (N == 4) {
      __builtin_amdgcn_raw_buffer_store_b16((uint16_t)mword, tile_rsrc(m_tile), code_off, 0, kNt);
      __builtin_amdgcn_raw_buffer_store_b16((uint16_t)vword, tile_rsrc(v_tile), code_off, 0, kNt);
    } else {
      __builtin_amdgcn_raw_buffer_store_b32(mword, tile_rsrc(m_tile), code_off, 0, kNt);
      __builtin_amdgcn_raw_buffer_store_b32(vword, tile_rsrc(v_tile), code_off, 0, kNt);
    }
  } else {
    const gptr<uint8_t> mb = as_global<uint8_t>(m_tile) + code_off;
    const gptr<uint8_t> vb = as_global<uint8_t>(v_tile) + code_off;
    const int nb = (nv + 1) >> 1;
#pragma unroll
    for (int k = 0; k < N / 2; ++k) {
      if (k < nb) {
        mb[k] = (uint8_t)(mword >> (8 * k));
        vb[k] = (uint8_t)(vword >> (8 * k));
      }
    }
  }
}

// The launch's gradient multiplier; false if the launch is to do nothing.
__device__ __forceinline__ bool grad_ops_begin(const GradOps &go, float &gscale) {
  if (go.skip && *as_global<const float>(go.skip) != 0.0f) return false;
  gscale = go.scale;
  if (go.scale_dev) gscale *= *as_global<const float>(go.scale_dev);
  return true;
}

template <bool PBF, bool GBF, bool EXT, bool SR>
__global__ __launch_bounds__(kThreads) void fused_4bit_kernel(const FusedArgs args) {
  using G = Geometry<PBF, GBF>;
  __shared__ uint2 lds[kLdsEntries];
  const int tid = threadIdx.x;
  const TableSlot slot = request_table_slot<SR>(tid);
  const uint32_t chunk = (blockIdx.x & 7u) * args.chunks_per_xcd + (blockIdx.x >> 3);
  if (chunk >= args.nchunks) return;  // whole workgroup: the grid is padded to a multiple of 8
  float gscale = 1.0f;
  if (EXT && !grad_ops_begin(args.go, gscale)) return;  // whole grid
  const bool zero_g = EXT && args.go.zero != 0u;
  const int t = find_tensor(args, chunk);
  const TensorDesc &T = args.desc[t];
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int64_t tile = (int64_t)(chunk - args.first_chunk[t]) * kWaves + wave;
  const int64_t begin = tile * G::kTile;
  if (begin >= T.numel) {  // wave past the end of the tensor: only help with the tables
    setup_tables<SR>(lds, tid, slot);
    return;
  }
  const uint32_t salt = SR ? args.sr_salt[t] : 0u;
  if (begin + G::kTile <= T.numel)
    process_tile<PBF, GBF, true, EXT, false, SR>(T, tile, lane, wave, tid, args.sc, lds, slot, gscale, zero_g, salt);
  else
    process_tile<PBF, GBF, false, EXT, false, SR>(T, tile, lane, wave, tid, args.sc, lds, slot, gscale, zero_g, salt);
}

// ---------------------------------------------------------------------------
// rank-1 scaling of the second moment: statistics, update, commit
// ---------------------------------------------------------------------------
constexpr int kStatRows = 64;            // rows per workgroup of the statistics kernel
constexpr int kStatColsPerWave = 512;    // 8 columns per lane
constexpr int kStatCols = kStatColsPerWave * kWaves;

__device__ __forceinline__ void atomic_max_nonneg(const float *addr, float x) {
  // non-negative floats order like their bit patterns
  atomicMax(reinterpret_cast<unsigned int *>(const_cast<float *>(addr)), f2bits(x));
}

// New second moments of a tile of kStatRows x kStatCols elements, reduced to row and
// column maxima (get_variance_tensor_statistics, adamw_fourbit_triton.py:738-746).  The
// arithmetic is the update kernel's, operation for operation, so the maxima are maxima
// of exactly the values that kernel quantizes.  Every lane keeps 8 columns over the
// tile's rows: one atomic per column per tile, one per row per wave.
template <bool GBF, bool EXT>
__global__ __launch_bounds__(kThreads) void rank1_stats_kernel(const Rank1StatArgs args) {
  constexpr int kAhead = 4;  // rows whose loads are in flight together
  // row maxima of each 16-lane quarter of each wave; reduced by the last phase
  __shared__ uint32_t row_bits[kWaves * 4][kStatRows];
  const uint32_t chunk = blockIdx.x;
  float gscale = 1.0f;
  if (EXT && !grad_ops_begin(args.go, gscale)) return;
  const int t = find_tensor(args, chunk);
  const auto &T = args.desc[t];
  const uint32_t local = chunk - args.first_chunk[t];
  const uint32_t groups = args.col_groups[t];
  const uint32_t rg = local / groups, cg = local - rg * groups;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int64_t col = (int64_t)cg * kStatCols + wave * kStatColsPerWave + lane * 8;
  const bool active = col < T.cols;  // cols is a multiple of 8: all 8 columns or none
  const int64_t row0 = (int64_t)rg * kStatRows;
  const int nrows = (int)(row0 + kStatRows < T.rows ? kStatRows : T.rows - row0);
  // lanes past the last column work on zeros: code 0 under a zero scale and a zero
  // gradient give a zero second moment, which leaves every maximum alone
  float c_old[8], c_max[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    c_old[k] = active ? as_global<const float>(T.cmax)[col + k] : 0.0f;
    c_max[k] = 0.0f;
  }
  const uint32_t quarter = (uint32_t)wave * 4u + ((uint32_t)lane >> 4);
  for (int r0 = 0; r0 < nrows; r0 += kAhead) {
    // a group past the tile's last row repeats that row: maxima do not mind
    u32x4 gw[kAhead][GBF ? 1 : 2];
    uint32_t vw[kAhead];
    float r_old[kAhead];
#pragma unroll
    for (int i = 0; i < kAhead; ++i) {
      const int r = r0 + i < nrows ? r0 + i : nrows - 1;
      const int64_t row = row0 + r;
      r_old[i] = as_global<const float>(T.rmax)[row];
      // row bases are uniform; the lane's column is a 32-bit offset
      const int64_t row_first = row * T.cols + ((int64_t)cg * kStatCols + wave * kStatColsPerWave);
      const uint32_t lane_elem = (uint32_t)lane * 8u;
      const void *g_row = static_cast<const char *>(T.g) + row_first * (GBF ? 2 : 4);
      const void *v_row = T.v + (row_first >> 1);
      vw[i] = 0u;
#pragma unroll
      for (int h = 0; h < (GBF ? 1 : 2); ++h) gw[i][h] = u32x4{0u, 0u, 0u, 0u};
      if (active) {
        vw[i] = __builtin_amdgcn_raw_buffer_load_b32(tile_rsrc(v_row), lane_elem >> 1, 0, kNtReadOnly);
        if (GBF) {
          gw[i][0] = __builtin_amdgcn_raw_buffer_load_b128(tile_rsrc(g_row), lane_elem * 2u, 0, kNtReadOnly);
        } else {
          gw[i][0] = __builtin_amdgcn_raw_buffer_load_b128(tile_rsrc(g_row), lane_elem * 4u, 0, kNtReadOnly);
          gw[i][GBF ? 0 : 1] = __builtin_amdgcn_raw_buffer_load_b128(tile_rsrc(g_row), lane_elem * 4u + 16u, 0, kNtReadOnly);
        }
      }
    }
#pragma unroll
    for (int i = 0; i < kAhead; ++i) {
      float g[8];
      if (GBF) {
        widen_bf16_pair(gw[i][0].x, g[0], g[1]);
        widen_bf16_pair(gw[i][0].y, g[2], g[3]);
        widen_bf16_pair(gw[i][0].z, g[4], g[5]);
        widen_bf16_pair(gw[i][0].w, g[6], g[7]);
      } else {
        const u32x4 lo = gw[i][0], hi = gw[i][GBF ? 0 : 1];
        g[0] = bits2f(lo.x); g[1] = bits2f(lo.y); g[2] = bits2f(lo.z); g[3] = bits2f(lo.w);
        g[4] = bits2f(hi.x); g[5] = bits2f(hi.y); g[6] = bits2f(hi.z); g[7] = bits2f(hi.w);
      }
      const uint32_t even = vw[i] & 0x0F0F0F0Fu, odd = (vw[i] >> 4) & 0x0F0F0F0Fu;  // one code per byte
      float r_max = 0.0f;
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const float gk = EXT ? g[k] * gscale : g[k];
        const uint32_t code = ((k & 1 ? odd : even) >> (8 * (k >> 1))) & 0xffu;
        const float code_value = __builtin_fmaf((float)code, 0.0625f, 0.0625f);  // (code + 1) / 16, exact
        const float v_old = code_value * __builtin_fminf(r_old[i], c_old[k]);
        const float v = args.b2 * v_old + args.r2 * (gk * gk);
        c_max[k] = __builtin_fmaxf(c_max[k], v);
        r_max = __builtin_fmaxf(r_max, v);
      }
      uint32_t u = f2bits(r_max);
      u = dpp_umax<0xB1>(u);
      u = dpp_umax<0x4E>(u);
      u = dpp_umax<0x141>(u);
      u = dpp_umax<0x140>(u);           // maximum of each 16-lane quarter, in all its lanes
      if ((lane & 15) == 0) row_bits[quarter][r0 + i] = u;   // slots past nrows are not read
    }
  }
  if (active) {
#pragma unroll
    for (int k = 0; k < 8; ++k)
      if (c_max[k] != 0.0f) atomic_max_nonneg(T.cmax_next + col + k, c_max[k]);
  }
  __syncthreads();
  if (tid < nrows) {
    uint32_t u = 0u;
#pragma unroll
    for (int qi = 0; qi < kWaves * 4; ++qi) u = u > row_bits[qi][tid] ? u : row_bits[qi][tid];
    if (u != 0u) atomic_max_nonneg(T.rmax_next + row0 + tid, bits2f(u));
  }
}

template <bool PBF, bool GBF, bool EXT>
__global__ __launch_bounds__(kThreads) void fused_4bit_rank1_kernel(const Rank1Args args) {
  using G = Geometry<PBF, GBF>;
  __shared__ uint2 lds[kLdsEntries];
  const int tid = threadIdx.x;
  const TableSlot slot = request_table_slot<false>(tid);
  const uint32_t chunk = (blockIdx.x & 7u) * args.chunks_per_xcd + (blockIdx.x >> 3);
  if (chunk >= args.nchunks) return;
  float gscale = 1.0f;
  if (EXT && !grad_ops_begin(args.go, gscale)) return;
  const bool zero_g = EXT && args.go.zero != 0u;
  const int t = find_tensor(args, chunk);
  const Rank1Desc &T = args.desc[t];
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int64_t tile = (int64_t)(chunk - args.first_chunk[t]) * kWaves + wave;
  const int64_t begin = tile * G::kTile;
  if (begin >= T.numel) {
    setup_tables<false>(lds, tid, slot);
    return;
  }
  if (begin + G::kTile <= T.numel)
    process_tile<PBF, GBF, true, EXT, true, false>(T, tile, lane, wave, tid, args.sc, lds, slot, gscale, zero_g, 0u);
  else
    process_tile<PBF, GBF, false, EXT, true, false>(T, tile, lane, wave, tid, args.sc, lds, slot, gscale, zero_g, 0u);
}

// After the update: the new statistics become the current ones and the buffers that
// received them go back to zero for the next step's maxima.  One workgroup column per
// tensor (blockIdx.y), grid-stride over rows + cols floats.
__global__ __launch_bounds__(256) void rank1_commit_kernel(const Rank1Args args) {
  float gscale;
  if (!grad_ops_begin(args.go, gscale)) return;
  const Rank1Desc &T = args.desc[blockIdx.y];
  const int64_t total = T.rows + T.cols;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const bool is_row = i < T.rows;
    const gptr<float> cur = as_global<float>(is_row ? T.rmax : T.cmax) + (is_row ? i : i - T.rows);
    const gptr<float> next = as_global<float>(is_row ? T.rmax_next : T.cmax_next) + (is_row ? i : i - T.rows);
    *cur = *next;
    *next = 0.0f;
  }
}

// Non-quantized step for small tensors (cuda_adamw_kernels.cu:100-133): fp32
// moments in place, same derived scalars and operation order as the fused path.
template <bool PBF, bool GBF, bool EXT>
__global__ __launch_bounds__(256) void single_tensor_kernel(const SmallArgs args) {
  const uint32_t chunk = blockIdx.x;
  float gscale = 1.0f;
  if (EXT && !grad_ops_begin(args.go, gscale)) return;
  const bool zero_g = EXT && args.go.zero != 0u;
  const int t = find_tensor(args, chunk);
  const SmallDesc &T = args.desc[t];
  const StepConsts &sc = args.sc;
  const int64_t base = (int64_t)(chunk - args.first_chunk[t]) * kSmallChunk;
  const int64_t end = base + kSmallChunk < T.numel ? base + kSmallChunk : T.numel;
  for (int64_t i = base + threadIdx.x; i < end; i += 256) {
    float gi = GBF ? bf16_bits_to_f32(as_global<const uint16_t>(T.g)[i])
                   : as_global<const float>(T.g)[i];
    if (EXT) {
      gi *= gscale;
      if (zero_g) {
        if (GBF) as_global<uint16_t>(const_cast<void *>(T.g))[i] = 0;
        else as_global<float>(const_cast<void *>(T.g))[i] = 0.0f;
      }
    }
    const float pi = PBF ? bf16_bits_to_f32(as_global<const uint16_t>(T.p)[i])
                         : as_global<const float>(T.p)[i];
    const float m = sc.b1 * as_global<const float>(T.m)[i] + sc.r1 * gi;
    const float v = sc.b2 * as_global<const float>(T.v)[i] + sc.r2 * (gi * gi);
    as_global<float>(T.m)[i] = m;
    as_global<float>(T.v)[i] = v;
    // exact form here: these tensors are tiny, so the divisions cost nothing
    const float den = __builtin_sqrtf(v) / sc.c2s + sc.eps;
    const float pn = pi * sc.wdu - sc.ss * (m / den);
    if (PBF) as_global<uint16_t>(T.p)[i] = (uint16_t)f32_to_bf16_bits(pn);
    else as_global<float>(T.p)[i] = pn;
  }
}


// ---------------------------------------------------------------------------
// global gradient norm (what a caller computes before it clips)
// ---------------------------------------------------------------------------
// Sum over a 256-thread workgroup in a fixed order; the result is valid in thread 0.
__device__ __forceinline__ double workgroup_sum(double x, double *lds4) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) x += __shfl_xor(x, off, 64);
  if ((threadIdx.x & 63) == 0) lds4[threadIdx.x >> 6] = x;
  __syncthreads();
  return (lds4[0] + lds4[1]) + (lds4[2] + lds4[3]);
}

// Squares are exact in fp64 and summed there: four accumulators per thread, chunks in
// grid-stride order, so the sum depends on the tensor list only, not on scheduling.
template <bool GBF>
__global__ __launch_bounds__(256) void grad_sumsq_kernel(const NormArgs args) {
  constexpr int kElemBytes = GBF ? 2 : 4;
  constexpr int64_t kChunkElems = kNormChunkBytes / kElemBytes;
  __shared__ double lds4[4];
  const int tid = threadIdx.x;
  double acc[4] = {0.0, 0.0, 0.0, 0.0};
  for (uint32_t chunk = blockIdx.x; chunk < args.nchunks; chunk += kNormPartials) {
    const int t = find_tensor(args, chunk);
    const NormDesc &T = args.desc[t];
    const int64_t base = (int64_t)(chunk - args.first_chunk[t]) * kChunkElems;
    const void *cb = static_cast<const char *>(T.g) + base * kElemBytes;
    const int64_t rem = T.numel - base;
    if (rem >= kChunkElems) {
      u32x4 w[8];
#pragma unroll
      for (int k = 0; k < 8; ++k)
        w[k] = __builtin_amdgcn_raw_buffer_load_b128(tile_rsrc(cb), (uint32_t)(k * 256 + tid) * 16u, 0, kNtReadOnly);
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const uint32_t u[4] = {w[k].x, w[k].y, w[k].z, w[k].w};
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          if (GBF) {
            float lo, hi;
            widen_bf16_pair(u[c], lo, hi);
            acc[c] = __builtin_fma((double)lo, (double)lo, acc[c]);
            acc[c] = __builtin_fma((double)hi, (double)hi, acc[c]);
          } else {
            const double x = (double)bits2f(u[c]);
            acc[c] = __builtin_fma(x, x, acc[c]);
          }
        }
      }
    } else {
      for (int64_t i = tid; i < rem; i += 256) {
        const double x = GBF ? (double)bf16_bits_to_f32(as_global<const uint16_t>(cb)[i])
                             : (double)as_global<const float>(cb)[i];
        acc[0] = __builtin_fma(x, x, acc[0]);
      }
    }
  }
  const double total = workgroup_sum((acc[0] + acc[1]) + (acc[2] + acc[3]), lds4);
  if (tid == 0) {
    const gptr<double> out = as_global<double>(args.partials) + blockIdx.x;
    *out = args.first ? total : *out + total;
  }
}

__global__ __launch_bounds__(256) void grad_norm_finish_kernel(const double *partials_, float scale,
                                                               const float *scale_dev, float max_norm,
                                                               float *out3_) {
  __shared__ double lds4[4];
  const gptr<const double> partials = as_global<const double>(partials_);
  double a = 0.0;
#pragma unroll
  for (int k = 0; k < kNormPartials / 256; ++k) a += partials[threadIdx.x * (kNormPartials / 256) + k];
  const double total = workgroup_sum(a, lds4);
  if (threadIdx.x == 0) {
    float s = scale;
    if (scale_dev) s *= *as_global<const float>(scale_dev);
    const float norm = __builtin_fabsf(s) * (float)__builtin_sqrt(total);
    // torch.nn.utils.clip_grad_norm_: max_norm / (total_norm + 1e-6), clamped to 1
    // (a NaN stays a NaN)
    float coef = 1.0f;
    if (max_norm > 0.0f) {
      coef = max_norm / (norm + 1e-6f);
      coef = coef > 1.0f ? 1.0f : coef;
    }
    const gptr<float> out3 = as_global<float>(out3_);
    out3[0] = norm;
    out3[1] = coef;
    out3[2] = s * coef;
  }
}

// ---------------------------------------------------------------------------
// stand-alone quantize / dequantize of one moment (checkpoint interchange)
// ---------------------------------------------------------------------------
// One wave per 128-element block, two elements (one packed byte) per lane.  These run
// once per checkpoint, so they take the exact route only: IEEE division and the
// 15-compare count (optim/adamw_fourbit_triton.py:618-630, cuda_adamw_kernels.cu:167-194).
template <bool SECOND>
__global__ __launch_bounds__(256) void quantize_kernel(const float *__restrict__ x_, int64_t numel,
                                                       uint8_t *__restrict__ codes_,
                                                       float *__restrict__ scale_) {
  const gptr<const float> x = as_global<const float>(x_);
  const int lane = threadIdx.x & 63;
  const int64_t blk = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t nblk = (numel + Q4ADAMW_BLOCK - 1) / Q4ADAMW_BLOCK;
  if (blk >= nblk) return;
  const int64_t e = blk * Q4ADAMW_BLOCK + lane * 2;
  const float a = e < numel ? x[e] : 0.0f;
  const float b = e + 1 < numel ? x[e + 1] : 0.0f;
  // fmaxf drops a NaN next to a number; two NaN count as 0: a NaN never becomes the scale
  const float lane_max = __builtin_fmaxf(__builtin_fabsf(a), __builtin_fabsf(b));
  uint32_t u = lane_max == lane_max ? f2bits(lane_max) : 0u;
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const uint32_t o = (uint32_t)__shfl_xor((int)u, off, 64);
    u = u > o ? u : o;
  }
  const float s = bits2f(u);
  if (lane == 0) as_global<float>(scale_)[blk] = s;
  if (e < numel) {
    uint32_t byte = 0;
    const float q0 = a / s, q1 = b / s;
#pragma unroll
    for (int k = 0; k < 15; ++k) {
      const float t = SECOND ? qmid_v(k) : bits2f(kQmidMBits[k]);
      byte += (t < q0) ? 1u : 0u;
      byte += (e + 1 < numel && t < q1) ? 16u : 0u;
    }
    as_global<uint8_t>(codes_)[e >> 1] = (uint8_t)byte;
  }
}

// Rank-1 forms for the second moment of a rows x cols matrix (run once per
// checkpoint).  Statistics: a workgroup takes 64 rows x 256 columns, a thread one
// column; row maxima meet in LDS, then one atomic per row and per column.
__global__ __launch_bounds__(256) void fill_zero_kernel(float *x_, int64_t n) {
  const gptr<float> x = as_global<float>(x_);
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) x[i] = 0.0f;
}

__global__ __launch_bounds__(256) void rank1_absmax_kernel(const float *x_, int64_t rows, int64_t cols,
                                                           float *row_max, float *col_max) {
  __shared__ uint32_t row_bits[64];
  const gptr<const float> x = as_global<const float>(x_);
  const int tid = threadIdx.x;
  const int64_t col = (int64_t)blockIdx.x * 256 + tid;
  const int64_t row0 = (int64_t)blockIdx.y * 64;
  const int nrows = (int)(row0 + 64 < rows ? 64 : rows - row0);
  if (tid < 64) row_bits[tid] = 0u;
  __syncthreads();
  float c_max = 0.0f;
  for (int r = 0; r < nrows; ++r) {
    float a = col < cols ? __builtin_fabsf(x[(row0 + r) * cols + col]) : 0.0f;
    a = a == a ? a : 0.0f;  // a NaN never becomes a maximum
    c_max = __builtin_fmaxf(c_max, a);
    uint32_t u = f2bits(a);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const uint32_t o = (uint32_t)__shfl_xor((int)u, off, 64);
      u = u > o ? u : o;
    }
    if ((tid & 63) == 0 && u != 0u) atomicMax(&row_bits[r], u);
  }
  if (col < cols && c_max != 0.0f) atomic_max_nonneg(col_max + col, c_max);
  __syncthreads();
  if (tid < nrows && row_bits[tid] != 0u) atomic_max_nonneg(row_max + row0 + tid, bits2f(row_bits[tid]));
}

// one thread per packed byte: x / min(row maximum, column maximum), IEEE division, the
// 15-compare count (optim/adamw_fourbit_triton.py:834-863)
__global__ __launch_bounds__(256) void quantize_rank1_kernel(const float *x_, int64_t rows, int64_t cols,
                                                             const float *row_max, const float *col_max,
                                                             uint8_t *codes_) {
  const int64_t e = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 2;
  if (e >= rows * cols) return;
  const int64_t i = e / cols, j = e - i * cols;  // cols is even: both elements in row i
  const float r = as_global<const float>(row_max)[i];
  uint32_t byte = 0;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const float q = as_global<const float>(x_)[e + h] / __builtin_fminf(r, as_global<const float>(col_max)[j + h]);
#pragma unroll
    for (int k = 0; k < 15; ++k) byte += (qmid_v(k) < q) ? (1u << (4 * h)) : 0u;
  }
  as_global<uint8_t>(codes_)[e >> 1] = (uint8_t)byte;
}

// optim/adamw_fourbit_triton.py:520-527: code-book entry times min(row, column maximum)
__global__ __launch_bounds__(256) void dequantize_rank1_kernel(const uint8_t *codes_, const float *row_max,
                                                               const float *col_max, int64_t rows,
                                                               int64_t cols, float *out_) {
  const int64_t e = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 2;
  if (e >= rows * cols) return;
  const int64_t i = e / cols, j = e - i * cols;
  const float r = as_global<const float>(row_max)[i];
  const uint32_t byte = as_global<const uint8_t>(codes_)[e >> 1];
  as_global<float>(out_)[e] = qmap_v((int)(byte & 15u)) * __builtin_fminf(r, as_global<const float>(col_max)[j]);
  as_global<float>(out_)[e + 1] = qmap_v((int)(byte >> 4)) * __builtin_fminf(r, as_global<const float>(col_max)[j + 1]);
}

// cuda_adamw_kernels.cu:329-343: code -> code-book entry * block scale
template <bool SECOND>
__global__ __launch_bounds__(256) void dequantize_kernel(const uint8_t *__restrict__ codes_,
                                                         const float *__restrict__ scale_,
                                                         int64_t numel, float *__restrict__ out_) {
  const int64_t e = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 2;
  if (e >= numel) return;
  const uint32_t byte = as_global<const uint8_t>(codes_)[e >> 1];
  const float s = as_global<const float>(scale_)[e / Q4ADAMW_BLOCK];
  const uint32_t c0 = byte & 15u, c1 = byte >> 4;
  const float v0 = (SECOND ? qmap_v((int)c0) : bits2f(kQmapMDev[c0])) * s;
  as_global<float>(out_)[e] = v0;
  if (e + 1 < numel) {
    const float v1 = (SECOND ? qmap_v((int)c1) : bits2f(kQmapMDev[c1])) * s;
    as_global<float>(out_)[e + 1] = v1;
  }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
static thread_local std::string g_err;

static int fail(int code, const std::string &msg) {
  g_err = msg;
  return code;
}

static int hip_fail(hipError_t e, const char *what) {
  g_err = std::string(what) + ": " + hipGetErrorString(e);
  return (int)e;
}

#define Q4_HIP(call)                                  \
  do {                                                \
    hipError_t e_ = (call);                           \
    if (e_ != hipSuccess) return hip_fail(e_, #call); \
  } while (0)

static int make_consts(float beta1, float beta2, float lr, float wd, float eps, float step,
                       StepConsts *out) {
  if (!(lr > 0.0f) || !(eps > 0.0f) || !(beta1 > 0.0f && beta1 < 1.0f) ||
      !(beta2 > 0.0f && beta2 < 1.0f) || !(wd >= 0.0f) || !(step >= 1.0f))
    return fail(Q4ADAMW_ERR_HYPER,
                "hyper-parameter out of range (need lr>0, eps>0, 0<beta<1, weight_decay>=0, step>=1)");
  float s[6];
  q4adamw_derive_scalars(beta1, beta2, lr, wd, step, s);
  out->b1 = beta1;
  out->b2 = beta2;
  out->r1 = s[4];
  out->r2 = s[5];
  out->wdu = s[3];
  out->ss = s[2];
  out->c2s = s[1];
  out->eps = eps;
  // a step size so small that these overflow moves no parameter: a zero scale with
  // an infinite offset makes the kernel's update term vanish
  const double den_scale = 1.0 / ((double)s[1] * (double)s[2]), den_eps = (double)eps / (double)s[2];
  const bool fits = den_scale <= (double)FLT_MAX && den_eps <= (double)FLT_MAX;
  out->den_scale = fits ? (float)den_scale : 0.0f;
  out->den_eps = fits ? (float)den_eps : INFINITY;
  return 0;
}

static bool aligned(const void *p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

static int check_dtypes(int p_dtype, int g_dtype) {
  if ((p_dtype != Q4ADAMW_FP32 && p_dtype != Q4ADAMW_BF16) ||
      (g_dtype != Q4ADAMW_FP32 && g_dtype != Q4ADAMW_BF16))
    return fail(Q4ADAMW_ERR_ARG, "dtype tag must be Q4ADAMW_FP32 or Q4ADAMW_BF16");
  return 0;
}

// Completes prefix and pivots of a launch batch and launches it.  Args is FusedArgs
// or SmallArgs; `chunks` is the batch's total chunk count.
template <typename Args>
static void finish_prefix(Args &a) {
  for (int i = a.ntensors; i < Args::kPivots * 8; ++i) a.first_chunk[i] = 0x7fffffffu;
  for (int k = 0; k < Args::kPivots; ++k) a.pivot[k] = a.first_chunk[k * 8];
}

static int launch_fused_batch(FusedArgs &a, uint64_t chunks, void (*kernel)(const FusedArgs),
                              hipStream_t stream) {
  finish_prefix(a);
  a.nchunks = (uint32_t)chunks;
  a.chunks_per_xcd = (uint32_t)((chunks + 7) / 8);
  hipLaunchKernelGGL(kernel, dim3(a.chunks_per_xcd * 8u), dim3(kThreads), 0, stream, a);
  Q4_HIP(hipGetLastError());
  return 0;
}

static int launch_small_batch(SmallArgs &a, uint64_t chunks, void (*kernel)(const SmallArgs),
                              hipStream_t stream) {
  finish_prefix(a);
  hipLaunchKernelGGL(kernel, dim3((unsigned)chunks), dim3(256), 0, stream, a);
  Q4_HIP(hipGetLastError());
  return 0;
}

typedef void (*FusedKernel)(const FusedArgs);
typedef void (*SmallKernel)(const SmallArgs);

template <bool EXT, bool SR>
static FusedKernel pick_fused_ext(bool pb, bool gb) {
  if (!pb && !gb) return fused_4bit_kernel<false, false, EXT, SR>;
  if (!pb && gb) return fused_4bit_kernel<false, true, EXT, SR>;
  if (pb && !gb) return fused_4bit_kernel<true, false, EXT, SR>;
  return fused_4bit_kernel<true, true, EXT, SR>;
}

// stochastic rounding comes with the gradient options' kernels only
static FusedKernel pick_fused(int p_dtype, int g_dtype, bool ext, bool sr = false) {
  const bool pb = p_dtype == Q4ADAMW_BF16, gb = g_dtype == Q4ADAMW_BF16;
  if (sr) return pick_fused_ext<true, true>(pb, gb);
  return ext ? pick_fused_ext<true, false>(pb, gb) : pick_fused_ext<false, false>(pb, gb);
}

template <bool EXT>
static SmallKernel pick_small_ext(bool pb, bool gb) {
  if (!pb && !gb) return single_tensor_kernel<false, false, EXT>;
  if (!pb && gb) return single_tensor_kernel<false, true, EXT>;
  if (pb && !gb) return single_tensor_kernel<true, false, EXT>;
  return single_tensor_kernel<true, true, EXT>;
}

static SmallKernel pick_small(int p_dtype, int g_dtype, bool ext) {
  const bool pb = p_dtype == Q4ADAMW_BF16, gb = g_dtype == Q4ADAMW_BF16;
  return ext ? pick_small_ext<true>(pb, gb) : pick_small_ext<false>(pb, gb);
}

typedef void (*Rank1Kernel)(const Rank1Args);
typedef void (*Rank1StatKernel)(const Rank1StatArgs);

template <bool EXT>
static Rank1Kernel pick_rank1_ext(bool pb, bool gb) {
  if (!pb && !gb) return fused_4bit_rank1_kernel<false, false, EXT>;
  if (!pb && gb) return fused_4bit_rank1_kernel<false, true, EXT>;
  if (pb && !gb) return fused_4bit_rank1_kernel<true, false, EXT>;
  return fused_4bit_rank1_kernel<true, true, EXT>;
}

static Rank1Kernel pick_rank1(int p_dtype, int g_dtype, bool ext) {
  const bool pb = p_dtype == Q4ADAMW_BF16, gb = g_dtype == Q4ADAMW_BF16;
  return ext ? pick_rank1_ext<true>(pb, gb) : pick_rank1_ext<false>(pb, gb);
}

static Rank1StatKernel pick_rank1_stats(int g_dtype, bool ext) {
  if (g_dtype == Q4ADAMW_BF16) return ext ? rank1_stats_kernel<true, true> : rank1_stats_kernel<true, false>;
  return ext ? rank1_stats_kernel<false, true> : rank1_stats_kernel<false, false>;
}

// Fills the kernels' view of the caller's gradient options; returns whether the
// launch needs the EXT kernels (false: the options change nothing).
static int make_grad_ops(const q4adamw_grad_options *opt, GradOps *go, bool *ext) {
  go->scale = 1.0f;
  go->zero = 0u;
  go->scale_dev = nullptr;
  go->skip = nullptr;
  *ext = false;
  if (!opt) return 0;
  if (opt->grad_scale_dev && (reinterpret_cast<uintptr_t>(opt->grad_scale_dev) & 3))
    return fail(Q4ADAMW_ERR_ALIGN, "grad_scale_dev must be 4-byte aligned");
  if (opt->skip_if_nonzero && (reinterpret_cast<uintptr_t>(opt->skip_if_nonzero) & 3))
    return fail(Q4ADAMW_ERR_ALIGN, "skip_if_nonzero must be 4-byte aligned");
  go->scale = opt->grad_scale;
  go->zero = opt->zero_grad ? 1u : 0u;
  go->scale_dev = opt->grad_scale_dev;
  go->skip = opt->skip_if_nonzero;
  *ext = opt->grad_scale != 1.0f || opt->zero_grad || opt->grad_scale_dev || opt->skip_if_nonzero;
  return 0;
}

constexpr uint64_t kMaxChunksPerLaunch = 0x7ffffff0ull;  // grid.x limit, with room for padding to 8

}  // namespace q4

using namespace q4;

static int fused_4bit_multi_impl(const q4adamw_tensor *tensors, int count, int p_dtype, int g_dtype,
                                 float beta1, float beta2, float lr, float weight_decay, float eps,
                                 float step, const q4adamw_grad_options *opt, bool sr,
                                 const uint32_t *salts, uint64_t seed, void *stream);

extern "C" {

void q4adamw_derive_scalars(float beta1, float beta2, float lr, float weight_decay, float step,
                            float *out6) {
  // volatile stores keep each operation an individually rounded fp32 operation
  volatile float pw1 = powf(beta1, step);
  volatile float pw2 = powf(beta2, step);
  volatile float c1 = 1.0f - pw1;
  volatile float om2 = 1.0f - pw2;
  volatile float lrwd = lr * weight_decay;
  out6[0] = c1;
  out6[1] = sqrtf(om2);
  out6[2] = lr / c1;
  out6[3] = 1.0f - lrwd;
  out6[4] = 1.0f - beta1;
  out6[5] = 1.0f - beta2;
}

void q4adamw_tables(int which, float *qmap16, float *qmid15) {
  for (int k = 0; k < 16; ++k) qmap16[k] = which ? qmap_v(k) : bits2f(kQmapMBits[k]);
  for (int k = 0; k < 15; ++k) qmid15[k] = which ? qmid_v(k) : bits2f(kQmidMBits[k]);
}

int q4adamw_mtable_entry(uint32_t index, uint32_t *out2) {
  if (index >= kMtabEntries || !out2) return fail(Q4ADAMW_ERR_ARG, "index out of range");
  const MtabEntry e = mtab_entry(index);
  out2[0] = e.lo;
  out2[1] = e.hi;
  return 0;
}

int q4adamw_mtable_half_bucket(uint32_t half_index) {
  if (half_index >= kHalfTableEntries) return fail(Q4ADAMW_ERR_ARG, "index out of range");
  return (int)half_index_bucket(half_index);
}

int q4adamw_fused_4bit_multi(const q4adamw_tensor *tensors, int count, int p_dtype, int g_dtype,
                             float beta1, float beta2, float lr, float weight_decay, float eps,
                             float step, void *stream) {
  return q4adamw_fused_4bit_multi_ex(tensors, count, p_dtype, g_dtype, beta1, beta2, lr,
                                     weight_decay, eps, step, nullptr, stream);
}

int q4adamw_fused_4bit_multi_ex(const q4adamw_tensor *tensors, int count, int p_dtype, int g_dtype,
                                float beta1, float beta2, float lr, float weight_decay, float eps,
                                float step, const q4adamw_grad_options *opt, void *stream) {
  return fused_4bit_multi_impl(tensors, count, p_dtype, g_dtype, beta1, beta2, lr, weight_decay, eps,
                               step, opt, false, nullptr, 0, stream);
}

int q4adamw_fused_4bit_multi_sr(const q4adamw_tensor *tensors, int count, const uint32_t *salts,
                                uint64_t seed, int p_dtype, int g_dtype, float beta1, float beta2,
                                float lr, float weight_decay, float eps, float step,
                                const q4adamw_grad_options *opt, void *stream) {
  return fused_4bit_multi_impl(tensors, count, p_dtype, g_dtype, beta1, beta2, lr, weight_decay, eps,
                               step, opt, true, salts, seed, stream);
}

uint32_t q4adamw_sr_tensor_salt(uint64_t seed, float step, uint32_t tensor_salt) {
  uint32_t h = lowbias32(tensor_salt);
  h = lowbias32(h ^ (uint32_t)step);
  h = lowbias32(h ^ (uint32_t)(seed >> 32));
  return lowbias32(h ^ (uint32_t)seed);
}

}  // extern "C"

static int fused_4bit_multi_impl(const q4adamw_tensor *tensors, int count, int p_dtype, int g_dtype,
                                 float beta1, float beta2, float lr, float weight_decay, float eps,
                                 float step, const q4adamw_grad_options *opt, bool sr,
                                 const uint32_t *salts, uint64_t seed, void *stream) {
  if (count < 0 || (count > 0 && !tensors)) return fail(Q4ADAMW_ERR_ARG, "bad tensor list");
  if (int rc = check_dtypes(p_dtype, g_dtype)) return rc;
  FusedArgs a;
  bool ext = false;
  if (int rc = make_consts(beta1, beta2, lr, weight_decay, eps, step, &a.sc)) return rc;
  if (int rc = make_grad_ops(opt, &a.go, &ext)) return rc;
  // a lane reads 8 consecutive elements at once when parameters and gradients are bf16, else 4
  const bool p_bf16 = p_dtype == Q4ADAMW_BF16;
  const bool wide = p_bf16 && g_dtype == Q4ADAMW_BF16;   // 8 elements per lane
  const int64_t chunk_elems = wide ? Geometry<true, true>::kChunk : Geometry<false, false>::kChunk;
  const uintptr_t p_align = 16, g_align = g_dtype == Q4ADAMW_BF16 ? (p_bf16 ? 16 : 8) : 16;
  const uintptr_t code_align = wide ? 4 : 2;
  // validate everything before the first launch
  for (int i = 0; i < count; ++i) {
    const q4adamw_tensor &t = tensors[i];
    if (t.numel < 0) return fail(Q4ADAMW_ERR_ARG, "negative numel");
    if (t.numel == 0) continue;
    if (!t.p || !t.g || !t.exp_avg || !t.exp_avg_sq || !t.exp_avg_scale || !t.exp_avg_sq_scale)
      return fail(Q4ADAMW_ERR_ARG, "null tensor pointer");
    if (!aligned(t.p, p_align) || !aligned(t.g, g_align))
      return fail(Q4ADAMW_ERR_ALIGN, "param and grad must be 16-byte aligned");
    if (!aligned(t.exp_avg, code_align) || !aligned(t.exp_avg_sq, code_align) ||
        !aligned(t.exp_avg_scale, 4) || !aligned(t.exp_avg_sq_scale, 4))
      return fail(Q4ADAMW_ERR_ALIGN, "code and scale buffers must be 4-byte aligned");
    if ((uint64_t)(t.numel + chunk_elems - 1) / chunk_elems > kMaxChunksPerLaunch)
      return fail(Q4ADAMW_ERR_TOO_LARGE, "tensor too large for one launch");
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const FusedKernel kernel = pick_fused(p_dtype, g_dtype, ext, sr);
  a.ntensors = 0;
  uint64_t chunks = 0;
  for (int i = 0; i < count; ++i) {
    const q4adamw_tensor &t = tensors[i];
    if (t.numel == 0) continue;
    const uint64_t c = (uint64_t)(t.numel + chunk_elems - 1) / chunk_elems;
    if (a.ntensors == kMaxTensors || chunks + c > kMaxChunksPerLaunch) {
      if (int rc = launch_fused_batch(a, chunks, kernel, s)) return rc;
      a.ntensors = 0;
      chunks = 0;
    }
    TensorDesc &d = a.desc[a.ntensors];
    d.p = t.p;
    d.g = t.g;
    d.m = t.exp_avg;
    d.v = t.exp_avg_sq;
    d.sm = t.exp_avg_scale;
    d.sv = t.exp_avg_sq_scale;
    d.numel = t.numel;
    a.sr_salt[a.ntensors] = sr ? q4adamw_sr_tensor_salt(seed, step, salts ? salts[i] : (uint32_t)i) : 0u;
    a.first_chunk[a.ntensors] = (uint32_t)chunks;
    ++a.ntensors;
    chunks += c;
  }
  if (a.ntensors > 0) return launch_fused_batch(a, chunks, kernel, s);
  return 0;
}

extern "C" {

int q4adamw_fused_4bit_rank1_multi(const q4adamw_rank1_tensor *tensors, int count, int p_dtype,
                                   int g_dtype, float beta1, float beta2, float lr,
                                   float weight_decay, float eps, float step,
                                   const q4adamw_grad_options *opt, void *stream) {
  if (count < 0 || (count > 0 && !tensors)) return fail(Q4ADAMW_ERR_ARG, "bad tensor list");
  if (int rc = check_dtypes(p_dtype, g_dtype)) return rc;
  Rank1Args a;
  Rank1StatArgs sa;
  bool ext = false;
  if (int rc = make_consts(beta1, beta2, lr, weight_decay, eps, step, &a.sc)) return rc;
  if (int rc = make_grad_ops(opt, &a.go, &ext)) return rc;
  sa.go = a.go;
  sa.b2 = a.sc.b2;
  sa.r2 = a.sc.r2;
  const bool p_bf16 = p_dtype == Q4ADAMW_BF16;
  const bool wide = p_bf16 && g_dtype == Q4ADAMW_BF16;   // 8 elements per lane
  const int64_t chunk_elems = wide ? Geometry<true, true>::kChunk : Geometry<false, false>::kChunk;
  for (int i = 0; i < count; ++i) {
    const q4adamw_rank1_tensor &t = tensors[i];
    if (t.rows < 0 || t.cols < 0) return fail(Q4ADAMW_ERR_ARG, "negative shape");
    if (t.rows == 0 || t.cols == 0) continue;
    if (t.cols % 8 != 0 || t.cols < 512)
      return fail(Q4ADAMW_ERR_ARG, "rank-1 scaling needs cols to be a multiple of 8 and at least 512");
    if (t.cols > 0x40000000ll || t.rows > 0x7ffffffffll / t.cols)
      return fail(Q4ADAMW_ERR_TOO_LARGE, "rank-1 scaling handles matrices of up to 2^35 - 1 elements");
    if (!t.p || !t.g || !t.exp_avg || !t.exp_avg_sq || !t.exp_avg_scale || !t.row_max || !t.col_max ||
        !t.row_max_next || !t.col_max_next)
      return fail(Q4ADAMW_ERR_ARG, "null tensor pointer");
    if (!aligned(t.p, 16) || !aligned(t.g, 16))
      return fail(Q4ADAMW_ERR_ALIGN, "param and grad must be 16-byte aligned");
    if (!aligned(t.exp_avg, 4) || !aligned(t.exp_avg_sq, 4) || !aligned(t.exp_avg_scale, 4) ||
        !aligned(t.row_max, 4) || !aligned(t.row_max_next, 4))
      return fail(Q4ADAMW_ERR_ALIGN, "code, scale and row buffers must be 4-byte aligned");
    if (!aligned(t.col_max, 16) || !aligned(t.col_max_next, 16))
      return fail(Q4ADAMW_ERR_ALIGN, "column buffers must be 16-byte aligned");
    const uint64_t numel = (uint64_t)t.rows * (uint64_t)t.cols;
    const uint64_t stat_chunks = (uint64_t)((t.rows + kStatRows - 1) / kStatRows) *
                                 (uint64_t)((t.cols + kStatCols - 1) / kStatCols);
    if ((numel + chunk_elems - 1) / chunk_elems > kMaxChunksPerLaunch || stat_chunks > kMaxChunksPerLaunch)
      return fail(Q4ADAMW_ERR_TOO_LARGE, "tensor too large for one launch");
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const Rank1Kernel kernel = pick_rank1(p_dtype, g_dtype, ext);
  const Rank1StatKernel stat_kernel = pick_rank1_stats(g_dtype, ext);
  a.ntensors = 0;
  uint64_t chunks = 0, stat_chunks = 0;
  // statistics of every tensor of the batch, then the update, then the commit
  auto launch = [&]() -> int {
    sa.ntensors = a.ntensors;
    finish_prefix(sa);
    sa.nchunks = (uint32_t)stat_chunks;
    hipLaunchKernelGGL(stat_kernel, dim3(sa.nchunks), dim3(kThreads), 0, s, sa);
    Q4_HIP(hipGetLastError());
    finish_prefix(a);
    a.nchunks = (uint32_t)chunks;
    a.chunks_per_xcd = (uint32_t)((chunks + 7) / 8);
    hipLaunchKernelGGL(kernel, dim3(a.chunks_per_xcd * 8u), dim3(kThreads), 0, s, a);
    Q4_HIP(hipGetLastError());
    hipLaunchKernelGGL(rank1_commit_kernel, dim3(64, (unsigned)a.ntensors), dim3(256), 0, s, a);
    Q4_HIP(hipGetLastError());
    a.ntensors = 0;
    chunks = 0;
    stat_chunks = 0;
    return 0;
  };
  for (int i = 0; i < count; ++i) {
    const q4adamw_rank1_tensor &t = tensors[i];
    if (t.rows == 0 || t.cols == 0) continue;
    const int64_t numel = t.rows * t.cols;
    const uint64_t c = (uint64_t)(numel + chunk_elems - 1) / chunk_elems;
    const uint32_t groups = (uint32_t)((t.cols + kStatCols - 1) / kStatCols);
    const uint64_t sc_ = (uint64_t)((t.rows + kStatRows - 1) / kStatRows) * groups;
    if (a.ntensors == kMaxRank1Tensors || chunks + c > kMaxChunksPerLaunch ||
        stat_chunks + sc_ > kMaxChunksPerLaunch) {
      if (int rc = launch()) return rc;
    }
    Rank1Desc &d = a.desc[a.ntensors];
    d.p = t.p;
    d.g = t.g;
    d.m = t.exp_avg;
    d.v = t.exp_avg_sq;
    d.sm = t.exp_avg_scale;
    d.rmax = t.row_max;
    d.cmax = t.col_max;
    d.rmax_next = t.row_max_next;
    d.cmax_next = t.col_max_next;
    d.numel = numel;
    d.rows = t.rows;
    d.cols = t.cols;
    const FastDiv fd = make_fast_div((uint32_t)(t.cols >> 3));
    d.div_magic = fd.magic;
    d.div_shift = fd.shift;
    a.first_chunk[a.ntensors] = (uint32_t)chunks;
    Rank1StatArgs::Desc &sd = sa.desc[a.ntensors];
    sd.g = t.g;
    sd.v = t.exp_avg_sq;
    sd.rmax = t.row_max;
    sd.cmax = t.col_max;
    sd.rmax_next = t.row_max_next;
    sd.cmax_next = t.col_max_next;
    sd.rows = t.rows;
    sd.cols = t.cols;
    sa.first_chunk[a.ntensors] = (uint32_t)stat_chunks;
    sa.col_groups[a.ntensors] = groups;
    ++a.ntensors;
    chunks += c;
    stat_chunks += sc_;
  }
  if (a.ntensors > 0) return launch();
  return 0;
}

int q4adamw_fused_4bit(void *p, const void *g, uint8_t *exp_avg, uint8_t *exp_avg_sq,
                       float *exp_avg_scale, float *exp_avg_sq_scale, int64_t numel, int p_dtype,
                       int g_dtype, float beta1, float beta2, float lr, float weight_decay,
                       float eps, float step, void *stream) {
  q4adamw_tensor t = {p, g, exp_avg, exp_avg_sq, exp_avg_scale, exp_avg_sq_scale, numel};
  return q4adamw_fused_4bit_multi(&t, 1, p_dtype, g_dtype, beta1, beta2, lr, weight_decay, eps,
                                  step, stream);
}

int q4adamw_fused_single_tensor_multi(const q4adamw_small_tensor *tensors, int count, int p_dtype,
                                      int g_dtype, float beta1, float beta2, float lr,
                                      float weight_decay, float eps, float step, void *stream) {
  return q4adamw_fused_single_tensor_multi_ex(tensors, count, p_dtype, g_dtype, beta1, beta2, lr,
                                              weight_decay, eps, step, nullptr, stream);
}

int q4adamw_fused_single_tensor_multi_ex(const q4adamw_small_tensor *tensors, int count,
                                         int p_dtype, int g_dtype, float beta1, float beta2,
                                         float lr, float weight_decay, float eps, float step,
                                         const q4adamw_grad_options *opt, void *stream) {
  if (count < 0 || (count > 0 && !tensors)) return fail(Q4ADAMW_ERR_ARG, "bad tensor list");
  if (int rc = check_dtypes(p_dtype, g_dtype)) return rc;
  SmallArgs a;
  bool ext = false;
  if (int rc = make_consts(beta1, beta2, lr, weight_decay, eps, step, &a.sc)) return rc;
  if (int rc = make_grad_ops(opt, &a.go, &ext)) return rc;
  const uintptr_t pa = p_dtype == Q4ADAMW_BF16 ? 2 : 4, ga = g_dtype == Q4ADAMW_BF16 ? 2 : 4;
  for (int i = 0; i < count; ++i) {
    const q4adamw_small_tensor &t = tensors[i];
    if (t.numel < 0) return fail(Q4ADAMW_ERR_ARG, "negative numel");
    if (t.numel == 0) continue;
    if (!t.p || !t.g || !t.exp_avg || !t.exp_avg_sq)
      return fail(Q4ADAMW_ERR_ARG, "null tensor pointer");
    if (!aligned(t.p, pa) || !aligned(t.g, ga) || !aligned(t.exp_avg, 4) || !aligned(t.exp_avg_sq, 4))
      return fail(Q4ADAMW_ERR_ALIGN, "tensor not aligned to its element size");
    if ((uint64_t)(t.numel + kSmallChunk - 1) / kSmallChunk > kMaxChunksPerLaunch)
      return fail(Q4ADAMW_ERR_TOO_LARGE, "tensor too large for one launch");
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const SmallKernel kernel = pick_small(p_dtype, g_dtype, ext);
  a.ntensors = 0;
  uint64_t chunks = 0;
  for (int i = 0; i < count; ++i) {
    const q4adamw_small_tensor &t = tensors[i];
    if (t.numel == 0) continue;
    const uint64_t c = (uint64_t)(t.numel + kSmallChunk - 1) / kSmallChunk;
    if (a.ntensors == kMaxSmallTensors || chunks + c > kMaxChunksPerLaunch) {
      if (int rc = launch_small_batch(a, chunks, kernel, s)) return rc;
      a.ntensors = 0;
      chunks = 0;
    }
    SmallDesc &d = a.desc[a.ntensors];
    d.p = t.p;
    d.g = t.g;
    d.m = t.exp_avg;
    d.v = t.exp_avg_sq;
    d.numel = t.numel;
    a.first_chunk[a.ntensors] = (uint32_t)chunks;
    ++a.ntensors;
    chunks += c;
  }
  if (a.ntensors > 0) return launch_small_batch(a, chunks, kernel, s);
  return 0;
}

int q4adamw_fused_single_tensor(void *p, const void *g, float *exp_avg, float *exp_avg_sq,
                                int64_t numel, int p_dtype, int g_dtype, float beta1, float beta2,
                                float lr, float weight_decay, float eps, float step,
                                void *stream) {
  q4adamw_small_tensor t = {p, g, exp_avg, exp_avg_sq, numel};
  return q4adamw_fused_single_tensor_multi(&t, 1, p_dtype, g_dtype, beta1, beta2, lr,
                                           weight_decay, eps, step, stream);
}

int q4adamw_grad_norm(const q4adamw_grad *grads, int count, int g_dtype, float grad_scale,
                      const float *grad_scale_dev, float max_norm, void *workspace,
                      size_t workspace_bytes, float *out3, void *stream) {
  if (count < 0 || (count > 0 && !grads)) return fail(Q4ADAMW_ERR_ARG, "bad tensor list");
  if (int rc = check_dtypes(Q4ADAMW_FP32, g_dtype)) return rc;
  if (!workspace || !out3) return fail(Q4ADAMW_ERR_ARG, "null workspace or output");
  if (workspace_bytes < Q4ADAMW_NORM_WORKSPACE_BYTES)
    return fail(Q4ADAMW_ERR_ARG, "workspace smaller than Q4ADAMW_NORM_WORKSPACE_BYTES");
  if (!aligned(workspace, 8) || !aligned(out3, 4) || (grad_scale_dev && !aligned(grad_scale_dev, 4)))
    return fail(Q4ADAMW_ERR_ALIGN, "workspace must be 8-byte, scalars 4-byte aligned");
  const bool bf16 = g_dtype == Q4ADAMW_BF16;
  const int64_t chunk_elems = kNormChunkBytes / (bf16 ? 2 : 4);
  for (int i = 0; i < count; ++i) {
    if (grads[i].numel < 0) return fail(Q4ADAMW_ERR_ARG, "negative numel");
    if (grads[i].numel == 0) continue;
    if (!grads[i].g) return fail(Q4ADAMW_ERR_ARG, "null tensor pointer");
    if (!aligned(grads[i].g, 16)) return fail(Q4ADAMW_ERR_ALIGN, "gradients must be 16-byte aligned");
    if ((uint64_t)(grads[i].numel + chunk_elems - 1) / chunk_elems > kMaxChunksPerLaunch)
      return fail(Q4ADAMW_ERR_TOO_LARGE, "tensor too large for one launch");
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  NormArgs a;
  a.partials = static_cast<double *>(workspace);
  a.first = 1u;
  a.ntensors = 0;
  uint64_t chunks = 0;
  auto launch = [&]() -> int {
    finish_prefix(a);
    a.nchunks = (uint32_t)chunks;
    if (bf16) hipLaunchKernelGGL(grad_sumsq_kernel<true>, dim3(kNormPartials), dim3(256), 0, s, a);
    else hipLaunchKernelGGL(grad_sumsq_kernel<false>, dim3(kNormPartials), dim3(256), 0, s, a);
    Q4_HIP(hipGetLastError());
    a.first = 0u;
    a.ntensors = 0;
    chunks = 0;
    return 0;
  };
  for (int i = 0; i < count; ++i) {
    if (grads[i].numel == 0) continue;
    const uint64_t c = (uint64_t)(grads[i].numel + chunk_elems - 1) / chunk_elems;
    if (a.ntensors == kMaxNormTensors || chunks + c > kMaxChunksPerLaunch) {
      if (int rc = launch()) return rc;
    }
    a.desc[a.ntensors].g = grads[i].g;
    a.desc[a.ntensors].numel = grads[i].numel;
    a.first_chunk[a.ntensors] = (uint32_t)chunks;
    ++a.ntensors;
    chunks += c;
  }
  // the first launch also defines every partial sum, so an empty list still takes one
  if (a.ntensors > 0 || a.first) {
    if (int rc = launch()) return rc;
  }
  hipLaunchKernelGGL(grad_norm_finish_kernel, dim3(1), dim3(256), 0, s,
                     static_cast<const double *>(workspace), grad_scale, grad_scale_dev, max_norm, out3);
  Q4_HIP(hipGetLastError());
  return 0;
}

int q4adamw_quantize(const float *x, int64_t numel, int which, uint8_t *codes, float *scales,
                     void *stream) {
  if (numel < 0 || (which != 0 && which != 1)) return fail(Q4ADAMW_ERR_ARG, "bad numel or moment selector");
  if (numel == 0) return 0;
  if (!x || !codes || !scales) return fail(Q4ADAMW_ERR_ARG, "null tensor pointer");
  if (!aligned(x, 4) || !aligned(scales, 4)) return fail(Q4ADAMW_ERR_ALIGN, "fp32 buffers must be 4-byte aligned");
  const uint64_t blocks = (uint64_t)(numel + Q4ADAMW_BLOCK - 1) / Q4ADAMW_BLOCK;
  const uint64_t grid = (blocks + 3) / 4;
  if (grid > kMaxChunksPerLaunch) return fail(Q4ADAMW_ERR_TOO_LARGE, "tensor too large for one launch");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (which) hipLaunchKernelGGL(quantize_kernel<true>, dim3((unsigned)grid), dim3(256), 0, s, x, numel, codes, scales);
  else hipLaunchKernelGGL(quantize_kernel<false>, dim3((unsigned)grid), dim3(256), 0, s, x, numel, codes, scales);
  Q4_HIP(hipGetLastError());
  return 0;
}

static int check_rank1_shape(int64_t rows, int64_t cols) {
  if (rows < 0 || cols < 0) return fail(Q4ADAMW_ERR_ARG, "negative shape");
  if (cols % 8 != 0) return fail(Q4ADAMW_ERR_ARG, "rank-1 scaling needs cols to be a multiple of 8");
  if (rows > 0 && cols > 0 && (cols > 0x40000000ll || rows > 0x7ffffffffll / cols))
    return fail(Q4ADAMW_ERR_TOO_LARGE, "rank-1 scaling handles matrices of up to 2^35 - 1 elements");
  return 0;
}

int q4adamw_quantize_rank1(const float *x, int64_t rows, int64_t cols, uint8_t *codes,
                           float *row_max, float *col_max, void *stream) {
  if (int rc = check_rank1_shape(rows, cols)) return rc;
  if (rows == 0 || cols == 0) return 0;
  if (!x || !codes || !row_max || !col_max) return fail(Q4ADAMW_ERR_ARG, "null tensor pointer");
  if (!aligned(x, 4) || !aligned(row_max, 4) || !aligned(col_max, 4))
    return fail(Q4ADAMW_ERR_ALIGN, "fp32 buffers must be 4-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(fill_zero_kernel, dim3(64), dim3(256), 0, s, row_max, rows);
  hipLaunchKernelGGL(fill_zero_kernel, dim3(64), dim3(256), 0, s, col_max, cols);
  const dim3 tiles((unsigned)((cols + 255) / 256), (unsigned)((rows + 63) / 64));
  if (tiles.y > 65535u) return fail(Q4ADAMW_ERR_TOO_LARGE, "more than 4194240 rows");
  hipLaunchKernelGGL(rank1_absmax_kernel, tiles, dim3(256), 0, s, x, rows, cols, row_max, col_max);
  const uint64_t grid = ((uint64_t)rows * cols / 2 + 255) / 256;
  hipLaunchKernelGGL(quantize_rank1_kernel, dim3((unsigned)grid), dim3(256), 0, s, x, rows, cols,
                     static_cast<const float *>(row_max), static_cast<const float *>(col_max), codes);
  Q4_HIP(hipGetLastError());
  return 0;
}

int q4adamw_dequantize_rank1(const uint8_t *codes, const float *row_max, const float *col_max,
                             int64_t rows, int64_t cols, float *out, void *stream) {
  if (int rc = check_rank1_shape(rows, cols)) return rc;
  if (rows == 0 || cols == 0) return 0;
  if (!codes || !row_max || !col_max || !out) return fail(Q4ADAMW_ERR_ARG, "null tensor pointer");
  if (!aligned(out, 4) || !aligned(row_max, 4) || !aligned(col_max, 4))
    return fail(Q4ADAMW_ERR_ALIGN, "fp32 buffers must be 4-byte aligned");
  const uint64_t grid = ((uint64_t)rows * cols / 2 + 255) / 256;
  hipLaunchKernelGGL(dequantize_rank1_kernel, dim3((unsigned)grid), dim3(256), 0,
                     static_cast<hipStream_t>(stream), codes, row_max, col_max, rows, cols, out);
  Q4_HIP(hipGetLastError());
  return 0;
}

int q4adamw_dequantize(const uint8_t *codes, const float *scales, int64_t numel, int which,
                       float *out, void *stream) {
  if (numel < 0 || (which != 0 && which != 1)) return fail(Q4ADAMW_ERR_ARG, "bad numel or moment selector");
  if (numel == 0) return 0;
  if (!out || !codes || !scales) return fail(Q4ADAMW_ERR_ARG, "null tensor pointer");
  if (!aligned(out, 4) || !aligned(scales, 4)) return fail(Q4ADAMW_ERR_ALIGN, "fp32 buffers must be 4-byte aligned");
  const uint64_t grid = ((uint64_t)(numel + 1) / 2 + 255) / 256;
  if (grid > kMaxChunksPerLaunch) return fail(Q4ADAMW_ERR_TOO_LARGE, "tensor too large for one launch");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (which) hipLaunchKernelGGL(dequantize_kernel<true>, dim3((unsigned)grid), dim3(256), 0, s, codes, scales, numel, out);
  else hipLaunchKernelGGL(dequantize_kernel<false>, dim3((unsigned)grid), dim3(256), 0, s, codes, scales, numel, out);
  Q4_HIP(hipGetLastError());
  return 0;
}

int q4adamw_release(void) { return 0; }

const char *q4adamw_last_error(void) { return g_err.c_str(); }

int q4adamw_version(void) { return 1006; }

}  // extern "C"
