// Fused 4-bit AdamW step for MI355X (gfx950): host launchers and the C ABI declared in
// include/q4adamw.h.  The kernels live in the headers this file includes:
//   q4adamw_tables.h  code books, thresholds, bucket and interval tables (constexpr)
//   q4adamw_args.h    kernel argument structs and the device copies of the tables
//   q4adamw_device.h  device helpers
//   q4adamw_step.h    the fused step (block-scaled, stochastic rounding, rank-1); its kernels are
//                     instantiated in q4adamw_pick_*.hip (q4adamw_pick.h)
//   q4adamw_rank1.h   rank-1 scaling: statistics, commit, folds
//   q4adamw_aux.h     small-tensor step, gradient norm, quantize / dequantize
//
// Build (quantfour_adamw_cuda_amd/build.py): every q4adamw*.hip is compiled by itself with
// hipcc --offload-arch=gfx950 -O3 -ffp-contract=off -fPIC -c, side by side, and the objects
// are linked into one shared library (-ffp-contract=off matters: the moment updates and the
// exact parameter update must be individually rounded fp32 operations; fused multiply-adds
// appear only where written out).
//
// Work decomposition of the fused kernel (shaped by measurement: HBM on this part
// streams best when every wave is short-lived, touches 1 KiB of the widest stream
// with ONE 16-byte access per lane, and every access is marked non-temporal)
//   tile    = one wave64, one pass; a lane owns 16 bytes of the widest of the parameter
//             and gradient streams: 4 consecutive elements (tile = 256 elements = 2
//             quantization blocks, a block = 32 lanes, abs-max by one v_permlane16_swap
//             plus four DPP row steps), or 8 when parameters and gradients are both
//             16-bit types (tile = 512 elements = 4 blocks, a block = one 16-lane DPP row).
//             No LDS traffic and no barrier in the reduction.
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

#include <atomic>
#include <string>

#include "../../include/q4adamw.h"
#include "q4adamw_args.h"
#include "q4adamw_aux.h"
#include "q4adamw_device.h"
#include "q4adamw_pick.h"
#include "q4adamw_rank1.h"
#include "q4adamw_step.h"
#include "q4adamw_tables.h"

namespace q4 {

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
  make_exact_consts(out);
  return 0;
}

static bool aligned(const void *p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

static int check_dtypes(int p_dtype, int g_dtype) {
  if (p_dtype < Q4ADAMW_FP32 || p_dtype > Q4ADAMW_FP16 || g_dtype < Q4ADAMW_FP32 || g_dtype > Q4ADAMW_FP16)
    return fail(Q4ADAMW_ERR_ARG, "dtype tag must be Q4ADAMW_FP32, Q4ADAMW_BF16 or Q4ADAMW_FP16");
  return 0;
}

// Completes prefix and pivots of a launch batch and launches it.  Args is FusedArgs
// or SmallArgs; `chunks` is the batch's total chunk count.
template <typename Args>
static void finish_prefix(Args &a) {
  for (int i = a.ntensors; i < Args::kPivots * 8; ++i) a.first_chunk[i] = 0x7fffffffu;
  for (int k = 0; k < Args::kPivots; ++k) a.pivot[k] = a.first_chunk[k * 8];
}

// Two limits.  A batch (one set of kernel arguments) indexes its chunks with 31 bits
// (first_chunk's sentinel is 0x7fffffff).  A grid is smaller: HIP refuses a launch whose
// gridDim.x * blockDim.x reaches 2^32 (hip_runtime_api.h, hipModuleLaunchKernel), i.e. more than
// 2^24 - 1 workgroups of 256 threads, which 1.7e10 fp32 elements exceed -- a flat FSDP
// parameter fits 288 GB several times over.  So a batch's chunks are dealt to as many grids as
// it takes, each with the number of its first chunk in the arguments (chunk_base); a tensor
// larger than a grid simply spans grids.  The grid size is rounded down to a multiple of 8 (the
// fused kernels pad their grids to one).
constexpr uint64_t kMaxChunksPerLaunch = 0x7ffffff0ull;   // per batch
constexpr uint64_t kHipWorkItemsPerGrid = 0xffffffffull;
constexpr int64_t kMaxInterchangeElements = 1ll << 40;     // q4adamw_quantize / q4adamw_dequantize
static std::atomic<uint64_t> g_grid_limit_override{0};    // q4adamw_set_grid_limit (tests)

static uint64_t grid_limit(unsigned threads) {
  const uint64_t hw = (kHipWorkItemsPerGrid / threads) & ~7ull;
  const uint64_t o = g_grid_limit_override.load(std::memory_order_relaxed) & ~7ull;
  return o >= 8 && o < hw ? o : hw;
}

// Calls launch(base, count) for the grids of a batch of `chunks` chunks.
template <typename F>
static int for_each_grid(uint64_t chunks, unsigned threads, F launch) {
  const uint64_t limit = grid_limit(threads);
  for (uint64_t base = 0; base < chunks; base += limit) {
    const uint64_t count = chunks - base < limit ? chunks - base : limit;
    if (int rc = launch(base, count)) return rc;
  }
  return 0;
}

static int launch_fused_batch(FusedArgs &a, uint64_t chunks, void (*kernel)(const FusedArgs),
                              hipStream_t stream) {
  finish_prefix(a);
  return for_each_grid(chunks, kThreads, [&](uint64_t base, uint64_t count) -> int {
    a.chunk_base = (uint32_t)base;
    a.nchunks = (uint32_t)(base + count);
    a.chunks_per_xcd = (uint32_t)((count + 7) / 8);
    hipLaunchKernelGGL(kernel, dim3(a.chunks_per_xcd * 8u), dim3(kThreads), 0, stream, a);
    Q4_HIP(hipGetLastError());
    return 0;
  });
}

static int launch_small_batch(SmallArgs &a, uint64_t chunks, void (*kernel)(const SmallArgs),
                              hipStream_t stream) {
  finish_prefix(a);
  return for_each_grid(chunks, 256, [&](uint64_t base, uint64_t count) -> int {
    a.chunk_base = (uint32_t)base;
    hipLaunchKernelGGL(kernel, dim3((unsigned)count), dim3(256), 0, stream, a);
    Q4_HIP(hipGetLastError());
    return 0;
  });
}

template <bool EXT>
static SmallKernel pick_small_ext(int p_dtype, int g_dtype) {
  Q4_PICK_PG(single_tensor_kernel, EXT)
}

static SmallKernel pick_small(int p_dtype, int g_dtype, bool ext) {
  return ext ? pick_small_ext<true>(p_dtype, g_dtype) : pick_small_ext<false>(p_dtype, g_dtype);
}

// Which of the three update kernels a matrix takes, in the order of the launch passes.
// Rows form: rows of a whole number of quantization blocks and at least two tiles, and enough
// rows that the waves left idle in the last group of four do not matter.  The last tile of a
// row may be a partial one as long as its idle lanes are at most a sixteenth of the row (they
// cost issue slots, which the 16-bit kernels have none to spare of; the wide form is 5 to 8 %
// slower than the rows form).
enum Rank1Shape { kShapeRows = 0, kShapeWide = 1, kShapeNarrow = 2, kShapeAny = 3 };

static Rank1Shape rank1_shape(const q4adamw_rank1_tensor &t, int64_t tile_elems) {
  // rows that are no multiple of 8 elements long, or shorter than 16: lanes no longer lie in
  // one row, and rows start inside a byte of the packed codes; every element finds its own place
  if (t.cols % 8 != 0 || t.cols < 16) return kShapeAny;
  if (t.cols < tile_elems) return kShapeNarrow;
  const int64_t padded = (t.cols + tile_elems - 1) / tile_elems * tile_elems;
  if (t.cols % Q4ADAMW_BLOCK == 0 && t.cols >= 2 * tile_elems && t.rows >= 64 && (padded - t.cols) * 16 <= t.cols) {
    // The rounding noise is keyed by an element's 64-bit index, whose high half the kernels take
    // per tile: a tile must not straddle a multiple of 2^32.  Tiles of the other forms start at
    // multiples of their length and never do; a tile of the rows form starts where its row
    // does, so a matrix of more than 2^32 elements whose rows are no whole number of tiles
    // takes the wide form.
    const bool may_straddle = t.rows * t.cols > 0xffffffffll && t.cols % tile_elems != 0;
    if (!may_straddle) return kShapeRows;
  }
  return kShapeWide;
}

static uint64_t rank1_tiles_per_row(const q4adamw_rank1_tensor &t, int64_t tile_elems) {
  return (uint64_t)((t.cols + tile_elems - 1) / tile_elems);
}

static uint64_t rank1_chunks(const q4adamw_rank1_tensor &t, int64_t tile_elems) {
  if (rank1_shape(t, tile_elems) == kShapeRows)
    return (uint64_t)((t.rows + kWaves - 1) / kWaves) * rank1_tiles_per_row(t, tile_elems);
  const uint64_t chunk_elems = (uint64_t)tile_elems * kWaves;
  return ((uint64_t)t.rows * (uint64_t)t.cols + chunk_elems - 1) / chunk_elems;
}

template <bool EXT>
static Rank1StatKernel pick_rank1_stats_ext(int g_dtype) {
  if (g_dtype == Q4ADAMW_BF16) return rank1_stats_kernel<Q4ADAMW_BF16, EXT>;
  if (g_dtype == Q4ADAMW_FP16) return rank1_stats_kernel<Q4ADAMW_FP16, EXT>;
  return rank1_stats_kernel<Q4ADAMW_FP32, EXT>;
}

static Rank1StatKernel pick_rank1_stats(int g_dtype, bool ext) {
  return ext ? pick_rank1_stats_ext<true>(g_dtype) : pick_rank1_stats_ext<false>(g_dtype);
}

template <bool EXT>
static Rank1StatKernel pick_rank1_stats_any_ext(int g_dtype) {
  if (g_dtype == Q4ADAMW_BF16) return rank1_stats_any_kernel<Q4ADAMW_BF16, EXT>;
  if (g_dtype == Q4ADAMW_FP16) return rank1_stats_any_kernel<Q4ADAMW_FP16, EXT>;
  return rank1_stats_any_kernel<Q4ADAMW_FP32, EXT>;
}

static Rank1StatKernel pick_rank1_stats_any(int g_dtype, bool ext) {
  return ext ? pick_rank1_stats_any_ext<true>(g_dtype) : pick_rank1_stats_any_ext<false>(g_dtype);
}

// tiles of the statistics launch of a matrix, by the form its rows allow
static uint64_t rank1_stat_chunks(const q4adamw_rank1_tensor &t, uint32_t *col_groups) {
  const bool any = t.cols % 8 != 0 || t.cols < 16;
  const int64_t tile_rows = any ? kAnyStatRows : kStatRows, tile_cols = any ? kAnyStatCols : kStatCols;
  const uint64_t groups = (uint64_t)((t.cols + tile_cols - 1) / tile_cols);
  if (col_groups) *col_groups = (uint32_t)groups;
  return (uint64_t)((t.rows + tile_rows - 1) / tile_rows) * groups;
}

// Fills the kernels' view of the caller's gradient options; returns whether the
// launch needs the EXT kernels (false: the options change nothing).
static int make_grad_ops(const q4adamw_grad_options *opt, GradOps *go, bool *ext, int *update_form) {
  go->scale = 1.0f;
  go->zero = 0u;
  go->scale_dev = nullptr;
  go->skip = nullptr;
  go->sc_dev = nullptr;
  *ext = false;
  *update_form = Q4ADAMW_UPDATE_AUTO;
  if (!opt) return 0;
  if (opt->update_form < Q4ADAMW_UPDATE_AUTO || opt->update_form > Q4ADAMW_UPDATE_FOLDED)
    return fail(Q4ADAMW_ERR_ARG, "update_form must be Q4ADAMW_UPDATE_AUTO, Q4ADAMW_UPDATE_EXACT or Q4ADAMW_UPDATE_FOLDED");
  *update_form = opt->update_form;
  if (opt->step_consts && (reinterpret_cast<uintptr_t>(opt->step_consts) & 15))
    return fail(Q4ADAMW_ERR_ALIGN, "step_consts must be 16-byte aligned");
  if (opt->grad_scale_dev && (reinterpret_cast<uintptr_t>(opt->grad_scale_dev) & 3))
    return fail(Q4ADAMW_ERR_ALIGN, "grad_scale_dev must be 4-byte aligned");
  if (opt->skip_if_nonzero && (reinterpret_cast<uintptr_t>(opt->skip_if_nonzero) & 3))
    return fail(Q4ADAMW_ERR_ALIGN, "skip_if_nonzero must be 4-byte aligned");
  go->scale = opt->grad_scale;
  go->zero = opt->zero_grad ? 1u : 0u;
  go->scale_dev = opt->grad_scale_dev;
  go->skip = opt->skip_if_nonzero;
  go->sc_dev = static_cast<const StepConsts *>(opt->step_consts);
  *ext = opt->grad_scale != 1.0f || opt->zero_grad || opt->grad_scale_dev || opt->skip_if_nonzero ||
         opt->step_consts;
  return 0;
}

// Whether a call takes the kernels whose parameter update rounds every operation as IEEE 754
// does.  Left to the library (Q4ADAMW_UPDATE_AUTO) that is the case where it costs under one
// per cent of the step: fp32 parameters in the block-scaled step with nearest rounding -- the
// reference's fused path itself (optim/cuda_adamw_kernels.cu:266-419).  Elsewhere the folded
// form runs unless the caller asks (16-bit parameters +9 %, stochastic rounding +10 %, rank-1
// scaling +5 % of step time on the Llama parameter sets).
static bool exact_update(int update_form, int p_dtype, bool sr, bool rank1) {
  if (update_form == Q4ADAMW_UPDATE_EXACT) return true;
  if (update_form == Q4ADAMW_UPDATE_FOLDED) return false;
  return p_dtype == Q4ADAMW_FP32 && !sr && !rank1;
}


}  // namespace q4

using namespace q4;

static int fused_4bit_multi_impl(const q4adamw_tensor *tensors, int count, int p_dtype, int g_dtype,
                                 float beta1, float beta2, float lr, float weight_decay, float eps,
                                 float step, const q4adamw_grad_options *opt, bool sr,
                                 const uint32_t *salts, uint64_t seed, void *stream);
static int fused_4bit_rank1_multi_impl(const q4adamw_rank1_tensor *tensors, int count, int p_dtype,
                                       int g_dtype, float beta1, float beta2, float lr,
                                       float weight_decay, float eps, float step,
                                       const q4adamw_grad_options *opt, bool sr, const uint32_t *salts,
                                       uint64_t seed, void *stream);

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

int q4adamw_sr_bucket_entry(uint32_t half_index, uint32_t *out2) {
  if (half_index >= kHalfTableEntries || !out2) return fail(Q4ADAMW_ERR_ARG, "index out of range");
  const SrEntry e = sr_entry(half_index);
  out2[0] = e.thr;
  out2[1] = e.base;
  return 0;
}

int q4adamw_sr_affine_entry(uint32_t k, float *out2) {
  if (k > 16u || !out2) return fail(Q4ADAMW_ERR_ARG, "index out of range");
  const SrAffine a = sr_affine_m(k);
  out2[0] = a.a;
  out2[1] = a.c;
  return 0;
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
  int update_form = Q4ADAMW_UPDATE_AUTO;
  if (int rc = make_consts(beta1, beta2, lr, weight_decay, eps, step, &a.sc)) return rc;
  if (int rc = make_grad_ops(opt, &a.go, &ext, &update_form)) return rc;
  a.seed_lo = (uint32_t)seed;
  a.seed_hi = (uint32_t)(seed >> 32);
  // a lane reads 8 consecutive elements at once when parameters and gradients are 16-bit types, else 4
  const bool p_half = p_dtype != Q4ADAMW_FP32, g_half = g_dtype != Q4ADAMW_FP32;
  const bool wide = p_half && g_half;   // 8 elements per lane
  const int64_t chunk_elems = wide ? Geometry<1, 1>::kChunk : Geometry<0, 0>::kChunk;
  // Parameters and gradients need the alignment of their element type only: the 16-byte
  // accesses of the kernels are legal at any such address (the memory pipeline runs in its
  // unaligned mode under ROCm; the compiler relies on the same for amdhsa targets).  A view at
  // an odd offset into a flat buffer costs nothing on the gradient side and 6 to 9 % more
  // time on the parameter side (lines shared between waves; see kNtSharedLines).
  const uintptr_t p_align = p_half ? 2 : 4, g_align = g_half ? 2 : 4;
  const uintptr_t code_align = wide ? 4 : 2;
  // validate everything before the first launch
  for (int i = 0; i < count; ++i) {
    const q4adamw_tensor &t = tensors[i];
    if (t.numel < 0) return fail(Q4ADAMW_ERR_ARG, "negative numel");
    if (t.numel == 0) continue;
    if (!t.p || !t.g || !t.exp_avg || !t.exp_avg_sq || !t.exp_avg_scale || !t.exp_avg_sq_scale)
      return fail(Q4ADAMW_ERR_ARG, "null tensor pointer");
    if (!aligned(t.p, p_align) || !aligned(t.g, g_align))
      return fail(Q4ADAMW_ERR_ALIGN, "param and grad must be aligned to their element size");
    if (!aligned(t.exp_avg, code_align) || !aligned(t.exp_avg_sq, code_align) ||
        !aligned(t.exp_avg_scale, 4) || !aligned(t.exp_avg_sq_scale, 4))
      return fail(Q4ADAMW_ERR_ALIGN, "code and scale buffers must be 4-byte aligned");
    if (((uint64_t)t.numel + (uint64_t)chunk_elems - 1) / (uint64_t)chunk_elems > kMaxChunksPerLaunch)
      return fail(Q4ADAMW_ERR_TOO_LARGE, "tensor too large: more than 2^31 - 16 chunks");
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const FusedKernel kernel = pick_fused(p_dtype, g_dtype, ext, sr, exact_update(update_form, p_dtype, sr, false));
  a.ntensors = 0;
  uint64_t chunks = 0;
  for (int i = 0; i < count; ++i) {
    const q4adamw_tensor &t = tensors[i];
    if (t.numel == 0) continue;
    const uint64_t c = ((uint64_t)t.numel + (uint64_t)chunk_elems - 1) / (uint64_t)chunk_elems;
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
    a.sr_salt[a.ntensors] = !sr ? 0u : a.go.sc_dev ? lowbias32(salts ? salts[i] : (uint32_t)i)
                                                     : q4adamw_sr_tensor_salt(seed, step, salts ? salts[i] : (uint32_t)i);
    a.first_chunk[a.ntensors] = (uint32_t)chunks;
    ++a.ntensors;
    chunks += c;
  }
  if (a.ntensors > 0) return launch_fused_batch(a, chunks, kernel, s);
  return 0;
}

static int fused_4bit_rank1_multi_impl(const q4adamw_rank1_tensor *tensors, int count, int p_dtype,
                                       int g_dtype, float beta1, float beta2, float lr,
                                       float weight_decay, float eps, float step,
                                       const q4adamw_grad_options *opt, bool sr, const uint32_t *salts,
                                       uint64_t seed, void *stream) {
  if (count < 0 || (count > 0 && !tensors)) return fail(Q4ADAMW_ERR_ARG, "bad tensor list");
  if (int rc = check_dtypes(p_dtype, g_dtype)) return rc;
  Rank1Args a;
  Rank1StatArgs sa;
  bool ext = false;
  int update_form = Q4ADAMW_UPDATE_AUTO;
  if (int rc = make_consts(beta1, beta2, lr, weight_decay, eps, step, &a.sc)) return rc;
  if (int rc = make_grad_ops(opt, &a.go, &ext, &update_form)) return rc;
  a.seed_lo = (uint32_t)seed;
  a.seed_hi = (uint32_t)(seed >> 32);
  sa.go = a.go;
  sa.b2 = a.sc.b2;
  sa.r2 = a.sc.r2;
  const bool wide = p_dtype != Q4ADAMW_FP32 && g_dtype != Q4ADAMW_FP32;   // 8 elements per lane
  const int64_t chunk_elems = wide ? Geometry<1, 1>::kChunk : Geometry<0, 0>::kChunk;
  for (int i = 0; i < count; ++i) {
    const q4adamw_rank1_tensor &t = tensors[i];
    if (t.rows < 0 || t.cols < 0) return fail(Q4ADAMW_ERR_ARG, "negative shape");
    if (t.rows == 0 || t.cols == 0) continue;
    if (t.cols < 2) return fail(Q4ADAMW_ERR_ARG, "rank-1 scaling needs at least 2 columns");
    if (t.cols > 0x40000000ll || t.rows > 0x7ffffffffll / t.cols)
      return fail(Q4ADAMW_ERR_TOO_LARGE, "rank-1 scaling handles matrices of up to 2^35 - 1 elements");
    if ((t.cols % 8 != 0 || t.cols < 16) && t.rows * t.cols > 0xffffffffll)
      return fail(Q4ADAMW_ERR_TOO_LARGE,
                  "rank-1 scaling of rows that are no multiple of 8 long (or shorter than 16) handles fewer than 2^32 elements");
    if (!t.p || !t.g || !t.exp_avg || !t.exp_avg_sq || !t.exp_avg_scale || !t.row_max || !t.col_max ||
        !t.row_max_next || !t.col_max_next)
      return fail(Q4ADAMW_ERR_ARG, "null tensor pointer");
    if (!aligned(t.p, p_dtype != Q4ADAMW_FP32 ? 2 : 4) || !aligned(t.g, g_dtype != Q4ADAMW_FP32 ? 2 : 4))
      return fail(Q4ADAMW_ERR_ALIGN, "param and grad must be aligned to their element size");
    if (!aligned(t.exp_avg, 4) || !aligned(t.exp_avg_sq, 4) || !aligned(t.exp_avg_scale, 4) ||
        !aligned(t.row_max, 4) || !aligned(t.row_max_next, 4))
      return fail(Q4ADAMW_ERR_ALIGN, "code, scale and row buffers must be 4-byte aligned");
    if (!aligned(t.col_max, 16) || !aligned(t.col_max_next, 16))
      return fail(Q4ADAMW_ERR_ALIGN, "column buffers must be 16-byte aligned");
    if (t.lead_dims < 0 || t.lead_dims > 3) return fail(Q4ADAMW_ERR_ARG, "lead_dims must be 0 to 3");
    if (t.lead_dims >= 2) {
      int64_t prod = 1;
      for (int j = 0; j < t.lead_dims; ++j) {
        if (t.lead_shape[j] < 1 || !t.lead_max[j] || !t.lead_max_next[j])
          return fail(Q4ADAMW_ERR_ARG, "leading dimensions need a positive size and their statistics");
        if (!aligned(t.lead_max[j], 4) || !aligned(t.lead_max_next[j], 4))
          return fail(Q4ADAMW_ERR_ALIGN, "leading statistics must be 4-byte aligned");
        prod *= t.lead_shape[j];
      }
      if (prod != t.rows) return fail(Q4ADAMW_ERR_ARG, "rows must be the product of the leading dimensions");
    }
    const uint64_t stat_chunks = rank1_stat_chunks(t, nullptr);
    if (rank1_chunks(t, chunk_elems / kWaves) > kMaxChunksPerLaunch || stat_chunks > kMaxChunksPerLaunch)
      return fail(Q4ADAMW_ERR_TOO_LARGE, "tensor too large: more than 2^31 - 16 chunks");
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t tile_elems = chunk_elems / kWaves;
  const bool exact = exact_update(update_form, p_dtype, sr, true);
  FoldArgs fa;   // the batch's tensors with several leading dimensions
  fa.go = a.go;
  fa.ntensors = 0;
  Rank1Kernel kernel = nullptr;
  Rank1StatKernel stat_kernel = nullptr;
  a.ntensors = 0;
  uint64_t chunks = 0, stat_chunks = 0;
  // statistics of every tensor of the batch, then the update, then the commit
  auto launch = [&]() -> int {
    sa.ntensors = a.ntensors;
    finish_prefix(sa);
    sa.nchunks = (uint32_t)stat_chunks;
    if (int rc = for_each_grid(stat_chunks, kThreads, [&](uint64_t base, uint64_t count) -> int {
          sa.chunk_base = (uint32_t)base;
          hipLaunchKernelGGL(stat_kernel, dim3((unsigned)count), dim3(kThreads), 0, s, sa);
          Q4_HIP(hipGetLastError());
          return 0;
        }))
      return rc;
    if (fa.ntensors > 0) {   // rows' maxima -> leading statistics -> rows' scales
      hipLaunchKernelGGL(rank1_fold_kernel<0>, dim3(64, (unsigned)fa.ntensors), dim3(256), 0, s, fa);
      hipLaunchKernelGGL(rank1_fold_kernel<1>, dim3(64, (unsigned)fa.ntensors), dim3(256), 0, s, fa);
      Q4_HIP(hipGetLastError());
    }
    finish_prefix(a);
    if (int rc = for_each_grid(chunks, kThreads, [&](uint64_t base, uint64_t count) -> int {
          a.chunk_base = (uint32_t)base;
          a.nchunks = (uint32_t)(base + count);
          a.chunks_per_xcd = (uint32_t)((count + 7) / 8);
          hipLaunchKernelGGL(kernel, dim3(a.chunks_per_xcd * 8u), dim3(kThreads), 0, s, a);
          Q4_HIP(hipGetLastError());
          return 0;
        }))
      return rc;
    hipLaunchKernelGGL(rank1_commit_kernel, dim3(64, (unsigned)a.ntensors), dim3(256), 0, s, a);
    Q4_HIP(hipGetLastError());
    if (fa.ntensors > 0) {
      hipLaunchKernelGGL(rank1_fold_kernel<2>, dim3(8, (unsigned)fa.ntensors), dim3(256), 0, s, fa);
      Q4_HIP(hipGetLastError());
      fa.ntensors = 0;
    }
    a.ntensors = 0;
    chunks = 0;
    stat_chunks = 0;
    return 0;
  };
  // three passes: matrices whose rows are whole tiles take the kernel whose workgroups share
  // the columns' maxima of four rows; other matrices with rows of at least a tile the one
  // that finds a tile's row on the scalar unit; narrower ones the one whose lanes find their own
  for (int shape = kShapeRows; shape <= kShapeAny; ++shape) {
    kernel = shape == kShapeRows     ? pick_rank1_rows(p_dtype, g_dtype, ext, sr, exact)
             : shape == kShapeWide   ? pick_rank1_wide(p_dtype, g_dtype, ext, sr, exact)
             : shape == kShapeNarrow ? pick_rank1_narrow(p_dtype, g_dtype, ext, sr, exact)
                                     : pick_rank1_any(p_dtype, g_dtype, ext, sr, exact);
    stat_kernel = shape == kShapeAny ? pick_rank1_stats_any(g_dtype, ext) : pick_rank1_stats(g_dtype, ext);
    for (int i = 0; i < count; ++i) {
      const q4adamw_rank1_tensor &t = tensors[i];
      if (t.rows == 0 || t.cols == 0 || rank1_shape(t, tile_elems) != shape) continue;
      const int64_t numel = t.rows * t.cols;
      const uint64_t c = rank1_chunks(t, tile_elems);
      uint32_t groups = 0;
      const uint64_t sc_ = rank1_stat_chunks(t, &groups);
      if (a.ntensors == kMaxRank1Tensors || chunks + c > kMaxChunksPerLaunch ||
          stat_chunks + sc_ > kMaxChunksPerLaunch || (t.lead_dims >= 2 && fa.ntensors == kMaxFoldTensors)) {
        if (int rc = launch()) return rc;
      }
      if (t.lead_dims >= 2) {
        FoldDesc &f = fa.desc[fa.ntensors++];
        f.row_next = t.row_max_next;
        f.rows = t.rows;
        f.dims = t.lead_dims;
        for (int j = 0; j < 3; ++j) {
          f.shape[j] = j < t.lead_dims ? t.lead_shape[j] : 1;
          f.cur[j] = j < t.lead_dims ? t.lead_max[j] : nullptr;
          f.next[j] = j < t.lead_dims ? t.lead_max_next[j] : nullptr;
        }
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
      // the divisor the tensor's kernel needs: tiles per row, cols, or cols / 8
      const FastDiv fd = make_fast_div(shape == kShapeRows  ? (uint32_t)rank1_tiles_per_row(t, tile_elems)
                                       : shape == kShapeAny ? (uint32_t)t.cols
                                                            : (uint32_t)(t.cols >> 3));
      d.div_magic = fd.magic;
      d.div_shift = fd.shift;
      a.sr_salt[a.ntensors] = !sr ? 0u : a.go.sc_dev ? lowbias32(salts ? salts[i] : (uint32_t)i)
                                                     : q4adamw_sr_tensor_salt(seed, step, salts ? salts[i] : (uint32_t)i);
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
    if (a.ntensors > 0) {
      if (int rc = launch()) return rc;
    }
  }
  return 0;
}

// ---------------------------------------------------------------------------
// global gradient norm
// ---------------------------------------------------------------------------
// Partial sums of q4adamw_grad_norm_static: one fp64 value per workgroup of the sum-of-squares
// launch, 16 KiB, held by every device the library runs on until the process ends.  In host
// code this name is not a device address; norm_scratch() asks the runtime for the current
// device's copy once and hands that pointer to the kernels.
static __device__ __align__(256) double g_norm_scratch[kNormPartials];

constexpr int kMaxDevices = 64;
static std::atomic<double *> g_norm_scratch_ptr[kMaxDevices];

static int norm_scratch(hipStream_t stream, double **out) {
  int dev = -1;
  Q4_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return fail(Q4ADAMW_ERR_ARG, "device ordinal beyond the scratch table");
  // every device has its own copy of the array: a stream of another device than the current
  // one would run the kernels there with this device's address
  if (stream != nullptr && stream != hipStreamPerThread) {
    hipDevice_t stream_dev = -1;
    Q4_HIP(hipStreamGetDevice(stream, &stream_dev));
    if (stream_dev != dev) return fail(Q4ADAMW_ERR_ARG, "the stream belongs to another device than the current one");
  }
  double *p = g_norm_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {   // first call on this device (two threads racing here find the same address)
    void *sym = nullptr;
    Q4_HIP(hipGetSymbolAddress(&sym, HIP_SYMBOL(g_norm_scratch)));
    if (!sym) return fail(Q4ADAMW_ERR_ARG, "the runtime returned no address for the scratch array");
    p = static_cast<double *>(sym);
    g_norm_scratch_ptr[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return 0;
}

// partials: kNormPartials doubles of device memory, 8-byte aligned; every one of them is
// written by the first launch before anything reads it, so its previous contents do not matter
static int grad_norm_impl(const q4adamw_grad *grads, int count, int g_dtype, float grad_scale,
                          const float *grad_scale_dev, float max_norm, double *partials, float *out3,
                          void *stream) {
  if (count < 0 || (count > 0 && !grads)) return fail(Q4ADAMW_ERR_ARG, "bad tensor list");
  if (int rc = check_dtypes(Q4ADAMW_FP32, g_dtype)) return rc;
  if (!out3) return fail(Q4ADAMW_ERR_ARG, "null workspace or output");
  if (!aligned(out3, 4) || (grad_scale_dev && !aligned(grad_scale_dev, 4)))
    return fail(Q4ADAMW_ERR_ALIGN, "workspace must be 8-byte, scalars 4-byte aligned");
  const int64_t chunk_elems = kNormChunkBytes / (g_dtype != Q4ADAMW_FP32 ? 2 : 4);
  for (int i = 0; i < count; ++i) {
    if (grads[i].numel < 0) return fail(Q4ADAMW_ERR_ARG, "negative numel");
    if (grads[i].numel == 0) continue;
    if (!grads[i].g) return fail(Q4ADAMW_ERR_ARG, "null tensor pointer");
    if (!aligned(grads[i].g, g_dtype != Q4ADAMW_FP32 ? 2 : 4))
      return fail(Q4ADAMW_ERR_ALIGN, "gradients must be aligned to their element size");
    if (((uint64_t)grads[i].numel + (uint64_t)chunk_elems - 1) / (uint64_t)chunk_elems > kMaxChunksPerLaunch)
      return fail(Q4ADAMW_ERR_TOO_LARGE, "tensor too large: more than 2^31 - 16 chunks");
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  NormArgs a;
  a.partials = partials;
  a.first = 1u;
  a.ntensors = 0;
  uint64_t chunks = 0;
  auto launch = [&]() -> int {
    finish_prefix(a);
    a.nchunks = (uint32_t)chunks;
    if (g_dtype == Q4ADAMW_BF16) hipLaunchKernelGGL(grad_sumsq_kernel<Q4ADAMW_BF16>, dim3(kNormPartials), dim3(256), 0, s, a);
    else if (g_dtype == Q4ADAMW_FP16) hipLaunchKernelGGL(grad_sumsq_kernel<Q4ADAMW_FP16>, dim3(kNormPartials), dim3(256), 0, s, a);
    else hipLaunchKernelGGL(grad_sumsq_kernel<Q4ADAMW_FP32>, dim3(kNormPartials), dim3(256), 0, s, a);
    Q4_HIP(hipGetLastError());
    a.first = 0u;
    a.ntensors = 0;
    chunks = 0;
    return 0;
  };
  for (int i = 0; i < count; ++i) {
    if (grads[i].numel == 0) continue;
    const uint64_t c = ((uint64_t)grads[i].numel + (uint64_t)chunk_elems - 1) / (uint64_t)chunk_elems;
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
  hipLaunchKernelGGL(grad_norm_finish_kernel, dim3(1), dim3(256), 0, s, static_cast<const double *>(partials),
                     grad_scale, grad_scale_dev, max_norm, out3);
  Q4_HIP(hipGetLastError());
  return 0;
}

extern "C" {

int q4adamw_fused_4bit_rank1_multi(const q4adamw_rank1_tensor *tensors, int count, int p_dtype,
                                   int g_dtype, float beta1, float beta2, float lr,
                                   float weight_decay, float eps, float step,
                                   const q4adamw_grad_options *opt, void *stream) {
  return fused_4bit_rank1_multi_impl(tensors, count, p_dtype, g_dtype, beta1, beta2, lr, weight_decay,
                                     eps, step, opt, false, nullptr, 0, stream);
}

int q4adamw_fused_4bit_rank1_multi_sr(const q4adamw_rank1_tensor *tensors, int count,
                                      const uint32_t *salts, uint64_t seed, int p_dtype, int g_dtype,
                                      float beta1, float beta2, float lr, float weight_decay,
                                      float eps, float step, const q4adamw_grad_options *opt,
                                      void *stream) {
  return fused_4bit_rank1_multi_impl(tensors, count, p_dtype, g_dtype, beta1, beta2, lr, weight_decay,
                                     eps, step, opt, true, salts, seed, stream);
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
  int update_form = Q4ADAMW_UPDATE_AUTO;   // this kernel's update is always the exact form
  if (int rc = make_consts(beta1, beta2, lr, weight_decay, eps, step, &a.sc)) return rc;
  if (int rc = make_grad_ops(opt, &a.go, &ext, &update_form)) return rc;
  const uintptr_t pa = p_dtype != Q4ADAMW_FP32 ? 2 : 4, ga = g_dtype != Q4ADAMW_FP32 ? 2 : 4;
  for (int i = 0; i < count; ++i) {
    const q4adamw_small_tensor &t = tensors[i];
    if (t.numel < 0) return fail(Q4ADAMW_ERR_ARG, "negative numel");
    if (t.numel == 0) continue;
    if (!t.p || !t.g || !t.exp_avg || !t.exp_avg_sq)
      return fail(Q4ADAMW_ERR_ARG, "null tensor pointer");
    if (!aligned(t.p, pa) || !aligned(t.g, ga) || !aligned(t.exp_avg, 4) || !aligned(t.exp_avg_sq, 4))
      return fail(Q4ADAMW_ERR_ALIGN, "tensor not aligned to its element size");
    if (((uint64_t)t.numel + (uint64_t)kSmallChunk - 1) / (uint64_t)kSmallChunk > kMaxChunksPerLaunch)
      return fail(Q4ADAMW_ERR_TOO_LARGE, "tensor too large: more than 2^31 - 16 chunks");
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const SmallKernel kernel = pick_small(p_dtype, g_dtype, ext);
  a.ntensors = 0;
  uint64_t chunks = 0;
  for (int i = 0; i < count; ++i) {
    const q4adamw_small_tensor &t = tensors[i];
    if (t.numel == 0) continue;
    const uint64_t c = ((uint64_t)t.numel + (uint64_t)kSmallChunk - 1) / (uint64_t)kSmallChunk;
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
  if (!workspace) return fail(Q4ADAMW_ERR_ARG, "null workspace or output");
  if (workspace_bytes < Q4ADAMW_NORM_WORKSPACE_BYTES)
    return fail(Q4ADAMW_ERR_ARG, "workspace smaller than Q4ADAMW_NORM_WORKSPACE_BYTES");
  if (!aligned(workspace, 8)) return fail(Q4ADAMW_ERR_ALIGN, "workspace must be 8-byte, scalars 4-byte aligned");
  return grad_norm_impl(grads, count, g_dtype, grad_scale, grad_scale_dev, max_norm,
                        static_cast<double *>(workspace), out3, stream);
}

int q4adamw_grad_norm_static(const q4adamw_grad *grads, int count, int g_dtype, float grad_scale,
                             const float *grad_scale_dev, float max_norm, float *out3, void *stream) {
  double *partials = nullptr;
  if (int rc = norm_scratch(static_cast<hipStream_t>(stream), &partials)) return rc;
  return grad_norm_impl(grads, count, g_dtype, grad_scale, grad_scale_dev, max_norm, partials, out3, stream);
}

int q4adamw_bias_table(float beta1, float beta2, int64_t first_step, int64_t count, float *out2) {
  if (!(beta1 > 0.0f && beta1 < 1.0f) || !(beta2 > 0.0f && beta2 < 1.0f))
    return fail(Q4ADAMW_ERR_HYPER, "hyper-parameter out of range (need 0<beta<1)");
  if (first_step < 1 || count < 0 || (count > 0 && !out2)) return fail(Q4ADAMW_ERR_ARG, "bad step range or null output");
  for (int64_t k = 0; k < count; ++k) {
    float s[6];
    q4adamw_derive_scalars(beta1, beta2, 1.0f, 0.0f, (float)(first_step + k), s);
    out2[2 * k] = s[0];
    out2[2 * k + 1] = s[1];
  }
  return 0;
}

int q4adamw_device_step(float *step_dev, const float *bias_table_dev, int64_t table_first_step,
                        int64_t table_steps, const float *lr_dev, float beta1, float beta2, float lr,
                        float weight_decay, float eps, const float *skip_if_nonzero, void *consts_dev,
                        void *stream) {
  StepConsts unused;
  if (int rc = make_consts(beta1, beta2, lr, weight_decay, eps, 1.0f, &unused)) return rc;
  if (!step_dev || !bias_table_dev || !consts_dev) return fail(Q4ADAMW_ERR_ARG, "null pointer");
  if (table_first_step < 1 || table_steps < 1) return fail(Q4ADAMW_ERR_ARG, "empty bias table");
  if (!aligned(step_dev, 4) || !aligned(bias_table_dev, 8) || (lr_dev && !aligned(lr_dev, 4)) ||
      (skip_if_nonzero && !aligned(skip_if_nonzero, 4)) || !aligned(consts_dev, 16))
    return fail(Q4ADAMW_ERR_ALIGN, "scalars must be 4-byte, the table 8-byte, the constants 16-byte aligned");
  hipLaunchKernelGGL(device_step_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream), step_dev,
                     bias_table_dev, table_first_step, table_steps, lr_dev, beta1, beta2, lr, weight_decay, eps,
                     skip_if_nonzero, static_cast<StepConsts *>(consts_dev));
  Q4_HIP(hipGetLastError());
  return 0;
}

int q4adamw_quantize(const float *x, int64_t numel, int which, uint8_t *codes, float *scales,
                     void *stream) {
  if (numel < 0 || (which != 0 && which != 1)) return fail(Q4ADAMW_ERR_ARG, "bad numel or moment selector");
  if (numel == 0) return 0;
  if (!x || !codes || !scales) return fail(Q4ADAMW_ERR_ARG, "null tensor pointer");
  if (!aligned(x, 4) || !aligned(scales, 4)) return fail(Q4ADAMW_ERR_ALIGN, "fp32 buffers must be 4-byte aligned");
  const uint64_t blocks = ((uint64_t)numel + Q4ADAMW_BLOCK - 1) / Q4ADAMW_BLOCK;
  const uint64_t groups = (blocks + 3) / 4;
  if (numel > kMaxInterchangeElements) return fail(Q4ADAMW_ERR_TOO_LARGE, "more than 2^40 elements");
  hipStream_t s = static_cast<hipStream_t>(stream);
  return for_each_grid(groups, 256, [&](uint64_t base, uint64_t count) -> int {
    if (which) hipLaunchKernelGGL(quantize_kernel<true>, dim3((unsigned)count), dim3(256), 0, s, x, numel, codes, scales, (int64_t)base);
    else hipLaunchKernelGGL(quantize_kernel<false>, dim3((unsigned)count), dim3(256), 0, s, x, numel, codes, scales, (int64_t)base);
    Q4_HIP(hipGetLastError());
    return 0;
  });
}

static int check_rank1_shape(int64_t rows, int64_t cols) {
  if (rows < 0 || cols < 0) return fail(Q4ADAMW_ERR_ARG, "negative shape");
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
  const dim3 tiles((unsigned)((cols + 255) / 256), (unsigned)((rows + 63) / 64));
  if (tiles.y > 65535u) return fail(Q4ADAMW_ERR_TOO_LARGE, "more than 4194240 rows");
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(fill_zero_kernel, dim3(64), dim3(256), 0, s, row_max, rows);
  hipLaunchKernelGGL(fill_zero_kernel, dim3(64), dim3(256), 0, s, col_max, cols);
  hipLaunchKernelGGL(rank1_absmax_kernel, tiles, dim3(256), 0, s, x, rows, cols, row_max, col_max);
  const uint64_t groups = (((uint64_t)rows * cols + 1) / 2 + 255) / 256;
  return for_each_grid(groups, 256, [&](uint64_t base, uint64_t count) -> int {
    hipLaunchKernelGGL(quantize_rank1_kernel, dim3((unsigned)count), dim3(256), 0, s, x, rows, cols,
                       static_cast<const float *>(row_max), static_cast<const float *>(col_max), codes, (int64_t)base);
    Q4_HIP(hipGetLastError());
    return 0;
  });
}

int q4adamw_quantize_rank1_scaled(const float *x, int64_t rows, int64_t cols, const float *row_scale,
                                  const float *col_max, uint8_t *codes, void *stream) {
  if (int rc = check_rank1_shape(rows, cols)) return rc;
  if (rows == 0 || cols == 0) return 0;
  if (!x || !codes || !row_scale || !col_max) return fail(Q4ADAMW_ERR_ARG, "null tensor pointer");
  if (!aligned(x, 4) || !aligned(row_scale, 4) || !aligned(col_max, 4))
    return fail(Q4ADAMW_ERR_ALIGN, "fp32 buffers must be 4-byte aligned");
  const uint64_t groups = (((uint64_t)rows * cols + 1) / 2 + 255) / 256;
  return for_each_grid(groups, 256, [&](uint64_t base, uint64_t count) -> int {
    hipLaunchKernelGGL(quantize_rank1_kernel, dim3((unsigned)count), dim3(256), 0, static_cast<hipStream_t>(stream), x,
                       rows, cols, row_scale, col_max, codes, (int64_t)base);
    Q4_HIP(hipGetLastError());
    return 0;
  });
}

int q4adamw_dequantize_rank1(const uint8_t *codes, const float *row_max, const float *col_max,
                             int64_t rows, int64_t cols, float *out, void *stream) {
  if (int rc = check_rank1_shape(rows, cols)) return rc;
  if (rows == 0 || cols == 0) return 0;
  if (!codes || !row_max || !col_max || !out) return fail(Q4ADAMW_ERR_ARG, "null tensor pointer");
  if (!aligned(out, 4) || !aligned(row_max, 4) || !aligned(col_max, 4))
    return fail(Q4ADAMW_ERR_ALIGN, "fp32 buffers must be 4-byte aligned");
  const uint64_t groups = (((uint64_t)rows * cols + 1) / 2 + 255) / 256;
  return for_each_grid(groups, 256, [&](uint64_t base, uint64_t count) -> int {
    hipLaunchKernelGGL(dequantize_rank1_kernel, dim3((unsigned)count), dim3(256), 0,
                       static_cast<hipStream_t>(stream), codes, row_max, col_max, rows, cols, out, (int64_t)base);
    Q4_HIP(hipGetLastError());
    return 0;
  });
}

int q4adamw_dequantize(const uint8_t *codes, const float *scales, int64_t numel, int which,
                       float *out, void *stream) {
  if (numel < 0 || (which != 0 && which != 1)) return fail(Q4ADAMW_ERR_ARG, "bad numel or moment selector");
  if (numel == 0) return 0;
  if (!out || !codes || !scales) return fail(Q4ADAMW_ERR_ARG, "null tensor pointer");
  if (!aligned(out, 4) || !aligned(scales, 4)) return fail(Q4ADAMW_ERR_ALIGN, "fp32 buffers must be 4-byte aligned");
  const uint64_t groups = (((uint64_t)numel + 1) / 2 + 255) / 256;
  if (numel > kMaxInterchangeElements) return fail(Q4ADAMW_ERR_TOO_LARGE, "more than 2^40 elements");
  hipStream_t s = static_cast<hipStream_t>(stream);
  return for_each_grid(groups, 256, [&](uint64_t base, uint64_t count) -> int {
    if (which) hipLaunchKernelGGL(dequantize_kernel<true>, dim3((unsigned)count), dim3(256), 0, s, codes, scales, numel, out, (int64_t)base);
    else hipLaunchKernelGGL(dequantize_kernel<false>, dim3((unsigned)count), dim3(256), 0, s, codes, scales, numel, out, (int64_t)base);
    Q4_HIP(hipGetLastError());
    return 0;
  });
}

int q4adamw_rank1_form(int64_t rows, int64_t cols, int both_16_bit) {
  if (rows <= 0 || cols <= 0 || cols > 0x40000000ll || rows > 0x7ffffffffll / cols)
    return fail(Q4ADAMW_ERR_ARG, "bad shape");
  q4adamw_rank1_tensor t = {};
  t.rows = rows;
  t.cols = cols;
  return (int)rank1_shape(t, both_16_bit ? Geometry<1, 1>::kTile : Geometry<0, 0>::kTile);
}

void q4adamw_set_grid_limit(uint64_t workgroups) { g_grid_limit_override.store(workgroups); }

int q4adamw_grid_plan(uint64_t chunks, int threads, uint64_t *bases, uint64_t *counts, int capacity) {
  if (threads < 64 || threads > 1024 || capacity < 0 || (capacity > 0 && (!bases || !counts)))
    return fail(Q4ADAMW_ERR_ARG, "bad workgroup size or output arrays");
  if (chunks > kMaxChunksPerLaunch) return fail(Q4ADAMW_ERR_TOO_LARGE, "more than 2^31 - 16 chunks");
  int n = 0;
  for_each_grid(chunks, (unsigned)threads, [&](uint64_t base, uint64_t count) -> int {
    if (n < capacity) {
      bases[n] = base;
      counts[n] = count;
    }
    ++n;
    return 0;
  });
  return n;
}

int q4adamw_rounding_selfcheck(uint64_t *counts6, void *stream) {
  if (!counts6) return fail(Q4ADAMW_ERR_ARG, "null output");
  if (!aligned(counts6, 8)) return fail(Q4ADAMW_ERR_ALIGN, "the counters must be 8-byte aligned");
  static_assert(sizeof(unsigned long long) == sizeof(uint64_t), "64-bit counters");
  hipLaunchKernelGGL(rounding_selfcheck_kernel, dim3(8192), dim3(256), 0, static_cast<hipStream_t>(stream),
                     reinterpret_cast<unsigned long long *>(counts6));
  Q4_HIP(hipGetLastError());
  return 0;
}

int q4adamw_release(void) { return 0; }

const char *q4adamw_last_error(void) { return g_err.c_str(); }

int q4adamw_version(void) { return 1015; }

}  // extern "C"
