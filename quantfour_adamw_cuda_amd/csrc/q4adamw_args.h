// Launch arguments of the kernels (passed by value in the kernarg segment) and the constant
// tables they read.  Shared by the kernels and the host launchers of q4adamw.hip.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

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
  // the fused kernel's parameter update in its folded form, p*wdu - m'/(sqrt(v')*den_scale +
  // den_eps), the step size folded into the denominator: 1/(c2s*ss) and eps/ss
  float den_scale, den_eps;
  // For the correctly rounded form of the update: RN(1 / c2s), which sqrt(v') is divided by
  // c2s with (div_by_reciprocal), and whether eps and c2s lie where that form's short
  // sequences hold (non-zero: 2^-60 <= eps <= 2^60, 2^-13 <= c2s <= 1; otherwise every lane
  // takes the general expansions).
  float c2s_rcp;
  uint32_t exact_short;
};

// (float)(1.0 / (double)c) is RN(1/c): rounding a quotient twice is harmless when the wide
// format has at least 2 * 24 + 2 bits (host and device: fp64 division is IEEE on both).
__host__ __device__ inline void make_exact_consts(StepConsts *sc) {
  sc->c2s_rcp = (float)(1.0 / (double)sc->c2s);
  sc->exact_short = (sc->eps >= 8.673617379884035e-19f && sc->eps <= 1.152921504606847e+18f &&
                     sc->c2s >= 1.220703125e-4f && sc->c2s <= 1.0f) ? 1u : 0u;
}

// What a launch does to the gradients besides reading them (kernels with EXT only).
struct GradOps {
  float scale;             // host part of the multiplier
  uint32_t zero;           // non-zero: overwrite the gradients with zeros once they are read
  const float *scale_dev;  // device part of the multiplier, or null
  const float *skip;       // device flag, or null: non-zero turns the launch into a no-op
  const StepConsts *sc_dev;  // the step's derived scalars in device memory (device_step_kernel), or null
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
  // A batch's chunks run in one grid or, beyond what a grid may hold, in several: this grid
  // takes chunks [chunk_base, nchunks), 8 * chunks_per_xcd workgroups.
  uint32_t chunk_base;
  uint32_t nchunks;
  uint32_t chunks_per_xcd; // ceil((nchunks - chunk_base) / 8)
  uint32_t pivot[kPivots];
  uint32_t first_chunk[kPivots * 8];
  TensorDesc desc[kMaxTensors];
  // stochastic rounding: the tensors' noise salts of this step; with a step number on the
  // device (go.sc_dev) the hash of each tensor's own salt, which the kernel carries on
  // through step number and seed
  uint32_t sr_salt[kMaxTensors];
  uint32_t seed_lo, seed_hi;
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
  uint32_t chunk_base;     // this grid's first chunk (workgroup 0)
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
  // division of a 32-bit number by cols / 8 (rows form of the update kernel: by the number
  // of tiles in a row) as multiply-high, add and shifts
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
  uint32_t chunk_base;     // as FusedArgs
  uint32_t nchunks;
  uint32_t chunks_per_xcd;
  uint32_t pivot[kPivots];
  uint32_t first_chunk[kPivots * 8];
  uint32_t sr_salt[kMaxRank1Tensors];   // stochastic rounding: as FusedArgs::sr_salt
  uint32_t seed_lo, seed_hi;
  Rank1Desc desc[kMaxRank1Tensors];
};

struct Rank1StatArgs {
  static constexpr int kCapacity = kMaxRank1Tensors;
  static constexpr int kPivots = (kMaxRank1Tensors + 7) / 8;
  float b2, r2;
  GradOps go;
  int ntensors;
  uint32_t chunk_base;     // this grid's first tile (workgroup 0)
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

// Rank-1 scaling of a tensor with two or three leading dimensions (its rows are their
// product): the statistics kernel leaves every flattened row's own maximum, these kernels
// reduce them to one statistic per leading dimension and hand the update kernel the rows'
// scales, the minimum over a row's leading statistics.
constexpr int kMaxFoldTensors = 16;

struct FoldDesc {  // 104 bytes
  float *row_next;   // in: the rows' own new maxima; out: the rows' new scales
  int64_t rows;
  int32_t dims;      // 2 or 3 leading dimensions
  int32_t pad_;
  int64_t shape[3];
  float *cur[3];     // current statistic of each leading dimension
  float *next[3];    // the step's new statistics (all zero between steps)
};

struct FoldArgs {
  GradOps go;
  int ntensors;
  FoldDesc desc[kMaxFoldTensors];
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

static_assert(sizeof(StepConsts) <= Q4ADAMW_STEP_CONSTS_BYTES, "the device copy of a step's scalars");
static_assert(sizeof(FusedArgs) <= 4096 && sizeof(SmallArgs) <= 4096 && sizeof(NormArgs) <= 4096 &&
                  sizeof(Rank1Args) <= 4096 && sizeof(Rank1StatArgs) <= 4096 && sizeof(FoldArgs) <= 4096,
              "kernel arguments are limited to 4 KiB");

// the first-moment bucket table (see q4adamw_tables.h), copied into LDS by every
// workgroup at start-up, one entry per thread
__device__ const HalfTable kHalfTable = make_half_table();
// stochastic rounding: code-book entries per bucket and the 17 intervals between them
__device__ const SrHalfTable kSrHalfTable = make_sr_half_table();
__device__ const SrIntervalTable kSrIntervals = make_sr_interval_table();
__device__ const SrAffineTable kSrAffine = make_sr_affine_table();
// first-moment code book for kernels that index it per lane
__device__ const uint32_t kQmapMDev[16] = {
    0xbf633333u, 0xbf29999au, 0xbee00000u, 0xbe59999au, 0xbd9eb852u, 0xbd051eb8u,
    0xbbb43958u, 0x00000000u, 0x3bb43958u, 0x3d051eb8u, 0x3d9eb852u, 0x3e59999au,
    0x3ee00000u, 0x3f29999au, 0x3f633333u, 0x3f800000u};

}  // namespace q4
