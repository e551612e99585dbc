// Fused 4-bit AdamW step for MI355X (gfx950): kernels, launchers and the C ABI
// declared in include/q4adamw.h.
//
// Build: hipcc --offload-arch=gfx950 -O3 -ffp-contract=off -shared -fPIC
// (-ffp-contract=off matters: the moment updates must be individually rounded
// fp32 multiplies and adds; fused multiply-adds appear only where written out).
//
// Work decomposition of the fused kernel
//   tile      = 512 consecutive elements = 4 quantization blocks, handled by one
//               wave64 in one pass: lane l owns elements [8l, 8l+8), so a block is
//               exactly one 16-lane DPP row and its abs-max needs four DPP steps,
//               no LDS and no barrier.
//   chunk     = 8 * tiles_per_wave consecutive tiles of ONE tensor, handled by one
//               512-thread workgroup; wave w takes tiles w, w+8, w+16, ...
//   launch    = all chunks of all tensors; a workgroup finds its tensor by binary
//               search over the per-tensor first-chunk prefix (scalar loads).
// Per element the kernel reads p, g and one nibble of each moment, and writes p
// and one nibble of each moment; per block it reads and writes two fp32 scales.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>
#include <string.h>

#include <algorithm>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/q4adamw.h"
#include "q4adamw_tables.h"

namespace q4 {

constexpr int kTile = 512;
constexpr int kWaves = 8;
constexpr int kThreads = kWaves * 64;
constexpr int kSmallThreads = 256;
constexpr int kSmallChunk = 4096;

struct TensorDesc {  // 64 bytes, device-visible
  void *p;
  const void *g;
  uint32_t *m;
  uint32_t *v;
  float *sm;
  float *sv;
  int64_t numel;
  int64_t chunk0;  // index of this tensor's first chunk in the launch
};

struct SmallDesc {  // 48 bytes
  void *p;
  const void *g;
  float *m;
  float *v;
  int64_t numel;
  int64_t chunk0;
};

// derived on the host exactly as optim/cuda_adamw_kernels.cu:435-440
struct StepConsts {
  float b1, b2, r1, r2;  // beta1, beta2, 1-beta1, 1-beta2
  float wdu, ss;         // 1 - lr*wd, lr / (1 - beta1^t)
  float c2s, inv_c2s;    // sqrt(1 - beta2^t) and its reciprocal
  float eps;
};

// ---------------------------------------------------------------------------
// device helpers
// ---------------------------------------------------------------------------
// Pointers that arrive inside a descriptor are generic; every tensor lives in
// global memory, so say so and get global_load/global_store instead of flat ones.
template <typename T>
using gptr = __attribute__((address_space(1))) T *;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <typename T>
__device__ __forceinline__ gptr<T> as_global(const void *p) {
  return (gptr<T>)(uintptr_t)p;
}

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_umax(uint32_t x) {
  const uint32_t y = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, CTRL, 0xf, 0xf, true);
  return x > y ? x : y;
}

// Max over the 16 lanes of a DPP row, result in every lane of the row.  The input
// is a non-negative float (an abs-max), so its bit pattern orders like an unsigned
// integer and the reduction is four v_max_u32 with a DPP operand.
__device__ __forceinline__ float row_max16(float x) {
  uint32_t u = f2bits(x);
  u = dpp_umax<0xB1>(u);   // quad_perm [1,0,3,2]
  u = dpp_umax<0x4E>(u);   // quad_perm [2,3,0,1]
  u = dpp_umax<0x141>(u);  // row_half_mirror
  u = dpp_umax<0x140>(u);  // row_mirror
  return bits2f(u);
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return bits2f(h << 16); }

__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {  // round to nearest even
  return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)f);
}

// eight consecutive elements starting at element index e0 (a multiple of 8)
template <bool BF, bool FULL>
__device__ __forceinline__ void load8(const void *base, int64_t e0, int nv, float (&x)[8]) {
  if (FULL) {
    if (BF) {
      const u32x4 w = *as_global<const u32x4>(static_cast<const uint16_t *>(base) + e0);
      x[0] = bits2f(w.x << 16); x[1] = bits2f(w.x & 0xffff0000u);
      x[2] = bits2f(w.y << 16); x[3] = bits2f(w.y & 0xffff0000u);
      x[4] = bits2f(w.z << 16); x[5] = bits2f(w.z & 0xffff0000u);
      x[6] = bits2f(w.w << 16); x[7] = bits2f(w.w & 0xffff0000u);
    } else {
      const gptr<const f32x4> q = as_global<const f32x4>(static_cast<const float *>(base) + e0);
      const f32x4 a = q[0], b = q[1];
      x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w;
      x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
    }
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      x[j] = 0.0f;
      if (j < nv) {
        x[j] = BF ? bf16_bits_to_f32(as_global<const uint16_t>(base)[e0 + j])
                  : as_global<const float>(base)[e0 + j];
      }
    }
  }
}

template <bool BF, bool FULL>
__device__ __forceinline__ void store8(void *base, int64_t e0, int nv, const float (&x)[8]) {
  if (FULL) {
    if (BF) {
      u32x4 w;
      w.x = f32_to_bf16_bits(x[0]) | (f32_to_bf16_bits(x[1]) << 16);
      w.y = f32_to_bf16_bits(x[2]) | (f32_to_bf16_bits(x[3]) << 16);
      w.z = f32_to_bf16_bits(x[4]) | (f32_to_bf16_bits(x[5]) << 16);
      w.w = f32_to_bf16_bits(x[6]) | (f32_to_bf16_bits(x[7]) << 16);
      *as_global<u32x4>(static_cast<uint16_t *>(base) + e0) = w;
    } else {
      const gptr<f32x4> q = as_global<f32x4>(static_cast<float *>(base) + e0);
      q[0] = f32x4{x[0], x[1], x[2], x[3]};
      q[1] = f32x4{x[4], x[5], x[6], x[7]};
    }
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (j < nv) {
        if (BF) as_global<uint16_t>(base)[e0 + j] = (uint16_t)f32_to_bf16_bits(x[j]);
        else as_global<float>(base)[e0 + j] = x[j];
      }
    }
  }
}

// Exact quantization of eight values of one state: IEEE division by the block
// scale, then the number of thresholds strictly below the quotient
// (cuda_adamw_kernels.cu:167-194 in closed form).  0/0 is NaN and gets code 0.
struct F8 {
  float x[8];
};

template <bool SECOND>
__device__ __noinline__ uint32_t quantize8_exact(F8 v, float scale) {
  uint32_t word = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
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

// ---------------------------------------------------------------------------
// one tile of one tensor
// ---------------------------------------------------------------------------
template <bool PBF, bool GBF, bool FULL>
__device__ __forceinline__ void process_tile(const TensorDesc &T, int64_t tile, int lane,
                                             const StepConsts &sc, const uint2 *mtab,
                                             const float *lds_qm, const float *lds_qv) {
  const int64_t numel = T.numel;
  const int64_t e0 = tile * kTile + (int64_t)lane * 8;
  int nv = 8;
  if (!FULL) {
    const int64_t rem = numel - e0;
    nv = rem >= 8 ? 8 : (rem > 0 ? (int)rem : 0);
  }
  const int64_t blk = e0 >> 7;
  const bool row_ok = FULL || (blk << 7) < numel;

  float p[8], g[8];
  load8<PBF, FULL>(T.p, e0, nv, p);
  load8<GBF, FULL>(T.g, e0, nv, g);
  uint32_t mw = 0, vw = 0;
  if (FULL) {
    mw = as_global<const uint32_t>(T.m)[e0 >> 3];
    vw = as_global<const uint32_t>(T.v)[e0 >> 3];
  } else {
    const gptr<const uint8_t> mb = as_global<const uint8_t>(T.m) + (e0 >> 1);
    const gptr<const uint8_t> vb = as_global<const uint8_t>(T.v) + (e0 >> 1);
    const int nb = (nv + 1) >> 1;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (k < nb) {
        mw |= (uint32_t)mb[k] << (8 * k);
        vw |= (uint32_t)vb[k] << (8 * k);
      }
    }
  }
  float sm_old = 0.0f, sv_old = 0.0f;
  if (row_ok) {
    sm_old = as_global<const float>(T.sm)[blk];
    sv_old = as_global<const float>(T.sv)[blk];
  }

  // dequantize, update moments and parameter (cuda_adamw_kernels.cu:334-351)
  F8 mn, vn;
  float am = 0.0f, av = 0.0f;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float m_old = lds_qm[(mw >> (4 * j)) & 15u] * sm_old;
    const float v_old = lds_qv[(vw >> (4 * j)) & 15u] * sv_old;
    const float gj = g[j];
    float m = sc.b1 * m_old + sc.r1 * gj;
    float v = sc.b2 * v_old + sc.r2 * (gj * gj);
    if (!FULL && j >= nv) { m = 0.0f; v = 0.0f; }
    // parameter: only this part may use the hardware's 1-ulp sqrt and reciprocal
    const float den = __builtin_fmaf(__builtin_amdgcn_sqrtf(v), sc.inv_c2s, sc.eps);
    const float upd = m * __builtin_amdgcn_rcpf(den);
    p[j] = __builtin_fmaf(-sc.ss, upd, p[j] * sc.wdu);
    mn.x[j] = m;
    vn.x[j] = v;
    am = __builtin_fmaxf(am, __builtin_fabsf(m));
    av = __builtin_fmaxf(av, v);
  }
  store8<PBF, FULL>(T.p, e0, nv, p);

  // block scales (exact: max is order independent)
  am = row_max16(am);
  av = row_max16(av);
  if (row_ok && (lane & 15) == 0) {
    as_global<float>(T.sm)[blk] = am;
    as_global<float>(T.sv)[blk] = av;
  }

  // fast quantization: multiply by a refined reciprocal, decide every code whose
  // quotient is clear of all thresholds, flag the rest
  const bool safe_m = am >= kScaleLo && am <= kScaleHi;
  const bool safe_v = av >= kScaleLo && av <= kScaleHi;
  const float rm = safe_m ? refined_rcp(am) : 0.0f;
  const float rv = safe_v ? refined_rcp(av) : 0.0f;
  bool redo = (!safe_m && am != 0.0f) || (!safe_v && av != 0.0f);
  uint32_t mword = 0, vword = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float qm = mn.x[j] * rm;
    const uint2 ent = mtab[f2bits(qm) >> 21];
    const bool above_hi = qm > bits2f(ent.y);
    const bool above_lo = qm > bits2f(ent.x);
    redo |= (above_hi != above_lo);
    mword |= ((ent.x & 15u) + (above_hi ? 1u : 0u)) << (4 * j);

    // second moment: thresholds at 16q = k + 0.5, k = 1..15
    const float a = __builtin_fmaf(vn.x[j] * rv, 16.0f, kVGuard - 0.5f);
    redo |= __builtin_amdgcn_fractf(a) < 2.0f * kVGuard;
    vword |= (uint32_t)(int)a << (4 * j);  // a > -1, so truncation gives 0 for a < 0
  }
  if (__builtin_expect(redo, 0)) {
    mword = quantize8_exact<false>(mn, am);
    vword = quantize8_exact<true>(vn, av);
  }
  if (am == 0.0f) mword = 0;  // 0/0: code 0 for the whole block
  if (!FULL) {
    const uint32_t keep = nv >= 8 ? 0xffffffffu : ((1u << (4 * nv)) - 1u);
    mword &= keep;
    vword &= keep;
  }

  if (FULL) {
    as_global<uint32_t>(T.m)[e0 >> 3] = mword;
    as_global<uint32_t>(T.v)[e0 >> 3] = vword;
  } else {
    const gptr<uint8_t> mb = as_global<uint8_t>(T.m) + (e0 >> 1);
    const gptr<uint8_t> vb = as_global<uint8_t>(T.v) + (e0 >> 1);
    const int nb = (nv + 1) >> 1;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (k < nb) {
        mb[k] = (uint8_t)(mword >> (8 * k));
        vb[k] = (uint8_t)(vword >> (8 * k));
      }
    }
  }
}

template <bool PBF, bool GBF>
__global__ __launch_bounds__(kThreads) void fused_4bit_kernel(
    const TensorDesc *__restrict__ descs, int ntensors, TensorDesc one, int tiles_per_wave,
    StepConsts sc) {
  __shared__ uint2 mtab[kMtabEntries];
  __shared__ float lds_qm[16];
  __shared__ float lds_qv[16];
  const int tid = threadIdx.x;
  for (int i = tid; i < (int)kMtabEntries; i += kThreads) {
    const MtabEntry e = mtab_entry((uint32_t)i);
    mtab[i] = make_uint2(e.lo, e.hi);
  }
  if (tid < 16) {
    lds_qm[tid] = bits2f(kQmapMBits[tid]);
    lds_qv[tid] = qmap_v(tid);
  }
  __syncthreads();

  const int64_t chunk = blockIdx.x;
  TensorDesc T = one;
  if (ntensors > 0) {
    int lo = 0, hi = ntensors - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (descs[mid].chunk0 <= chunk) lo = mid; else hi = mid - 1;
    }
    T = descs[lo];
  }
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int64_t ntiles = (T.numel + kTile - 1) / kTile;
  const int64_t tile0 = (chunk - T.chunk0) * (int64_t)(kWaves * tiles_per_wave) + wave;
  for (int k = 0; k < tiles_per_wave; ++k) {
    const int64_t tile = tile0 + (int64_t)k * kWaves;
    if (tile >= ntiles) break;
    if ((tile + 1) * kTile <= T.numel) process_tile<PBF, GBF, true>(T, tile, lane, sc, mtab, lds_qm, lds_qv);
    else process_tile<PBF, GBF, false>(T, tile, lane, sc, mtab, lds_qm, lds_qv);
  }
}

// Non-quantized step for small tensors (cuda_adamw_kernels.cu:100-133): fp32
// moments in place, same derived scalars and operation order as the fused path.
template <bool PBF, bool GBF>
__global__ __launch_bounds__(kSmallThreads) void single_tensor_kernel(
    const SmallDesc *__restrict__ descs, int ntensors, SmallDesc one, StepConsts sc) {
  const int64_t chunk = blockIdx.x;
  SmallDesc T = one;
  if (ntensors > 0) {
    int lo = 0, hi = ntensors - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (descs[mid].chunk0 <= chunk) lo = mid; else hi = mid - 1;
    }
    T = descs[lo];
  }
  const int64_t base = (chunk - T.chunk0) * kSmallChunk;
  const int64_t end = base + kSmallChunk < T.numel ? base + kSmallChunk : T.numel;
  for (int64_t i = base + threadIdx.x; i < end; i += kSmallThreads) {
    const float gi = GBF ? bf16_bits_to_f32(as_global<const uint16_t>(T.g)[i])
                         : as_global<const float>(T.g)[i];
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
  out->inv_c2s = 1.0f / s[1];
  out->eps = eps;
  return 0;
}

static bool aligned(const void *p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// Device copies of descriptor tables.  A small ring per device: a table whose
// bytes equal what a slot already holds is not uploaded again; a slot is only
// overwritten after the last launch that read it has finished.
struct Slot {
  void *dev = nullptr;
  void *host = nullptr;  // pinned staging
  size_t cap = 0;
  hipEvent_t done = nullptr;
  bool pending = false;
  std::vector<char> content;
};
struct DevCache {
  int device = -1;
  Slot slots[4];
  int next = 0;
};
static std::mutex g_mu;
static std::vector<DevCache *> g_caches;

static DevCache *cache_for(int device) {
  for (DevCache *c : g_caches)
    if (c->device == device) return c;
  DevCache *c = new DevCache();
  c->device = device;
  g_caches.push_back(c);
  return c;
}

// returns the device address of a copy of blob; *slot_out is the slot to mark
static int stage_table(const void *blob, size_t bytes, hipStream_t stream, void **dev_out,
                       Slot **slot_out) {
  int device = 0;
  Q4_HIP(hipGetDevice(&device));
  DevCache *c = cache_for(device);
  for (Slot &s : c->slots) {
    if (s.dev && s.content.size() == bytes && memcmp(s.content.data(), blob, bytes) == 0) {
      *dev_out = s.dev;
      *slot_out = &s;
      return 0;
    }
  }
  Slot &s = c->slots[c->next];
  c->next = (c->next + 1) % 4;
  if (s.pending) {
    Q4_HIP(hipEventSynchronize(s.done));
    s.pending = false;
  }
  if (s.cap < bytes) {
    if (s.dev) Q4_HIP(hipFree(s.dev));
    if (s.host) Q4_HIP(hipHostFree(s.host));
    s.dev = s.host = nullptr;
    s.cap = 0;
    s.content.clear();
    const size_t cap = std::max<size_t>(bytes * 2, 4096);
    Q4_HIP(hipMalloc(&s.dev, cap));
    Q4_HIP(hipHostMalloc(&s.host, cap, hipHostMallocDefault));
    s.cap = cap;
  }
  if (!s.done) Q4_HIP(hipEventCreateWithFlags(&s.done, hipEventDisableTiming));
  memcpy(s.host, blob, bytes);
  s.content.assign(static_cast<const char *>(blob), static_cast<const char *>(blob) + bytes);
  Q4_HIP(hipMemcpyAsync(s.dev, s.host, bytes, hipMemcpyHostToDevice, stream));
  *dev_out = s.dev;
  *slot_out = &s;
  return 0;
}

static int mark_slot(Slot *s, hipStream_t stream) {
  Q4_HIP(hipEventRecord(s->done, stream));
  s->pending = true;
  return 0;
}

static int pick_tiles_per_wave(int64_t total_tiles) {
  // keep at least ~16 workgroups per CU in the launch before lengthening chunks
  int tpw = 8;
  while (tpw > 1 && total_tiles / (kWaves * tpw) < 4096) tpw >>= 1;
  return tpw;
}

template <typename K>
static void launch_fused(K kernel, int64_t grid, hipStream_t stream, const TensorDesc *dev,
                         int n, const TensorDesc &one, int tpw, const StepConsts &sc) {
  hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(kThreads), 0, stream, dev, n, one, tpw, sc);
}

static int run_fused(std::vector<TensorDesc> &descs, int p_dtype, int g_dtype,
                     const StepConsts &sc, hipStream_t stream) {
  int64_t total_tiles = 0;
  for (const TensorDesc &d : descs) total_tiles += (d.numel + kTile - 1) / kTile;
  if (total_tiles == 0) return 0;
  const int tpw = pick_tiles_per_wave(total_tiles);
  int64_t chunks = 0;
  for (TensorDesc &d : descs) {
    d.chunk0 = chunks;
    const int64_t tiles = (d.numel + kTile - 1) / kTile;
    chunks += (tiles + kWaves * tpw - 1) / (kWaves * tpw);
  }
  if (chunks > 0x7fffffffLL) return fail(Q4ADAMW_ERR_TOO_LARGE, "too many chunks for one launch");

  const TensorDesc *dev = nullptr;
  int n = 0;
  Slot *slot = nullptr;
  TensorDesc one = descs[0];
  std::unique_lock<std::mutex> lock(g_mu, std::defer_lock);
  if (descs.size() > 1) {
    lock.lock();
    void *d = nullptr;
    const int rc = stage_table(descs.data(), descs.size() * sizeof(TensorDesc), stream, &d, &slot);
    if (rc) return rc;
    dev = static_cast<const TensorDesc *>(d);
    n = (int)descs.size();
  }
  const bool pb = p_dtype == Q4ADAMW_BF16, gb = g_dtype == Q4ADAMW_BF16;
  if (!pb && !gb) launch_fused(fused_4bit_kernel<false, false>, chunks, stream, dev, n, one, tpw, sc);
  else if (!pb && gb) launch_fused(fused_4bit_kernel<false, true>, chunks, stream, dev, n, one, tpw, sc);
  else if (pb && !gb) launch_fused(fused_4bit_kernel<true, false>, chunks, stream, dev, n, one, tpw, sc);
  else launch_fused(fused_4bit_kernel<true, true>, chunks, stream, dev, n, one, tpw, sc);
  Q4_HIP(hipGetLastError());
  if (slot) return mark_slot(slot, stream);
  return 0;
}

template <typename K>
static void launch_small(K kernel, int64_t grid, hipStream_t stream, const SmallDesc *dev, int n,
                         const SmallDesc &one, const StepConsts &sc) {
  hipLaunchKernelGGL(kernel, dim3((unsigned)grid), dim3(kSmallThreads), 0, stream, dev, n, one, sc);
}

static int run_small(std::vector<SmallDesc> &descs, int p_dtype, int g_dtype, const StepConsts &sc,
                     hipStream_t stream) {
  int64_t chunks = 0;
  for (SmallDesc &d : descs) {
    d.chunk0 = chunks;
    chunks += (d.numel + kSmallChunk - 1) / kSmallChunk;
  }
  if (chunks == 0) return 0;
  if (chunks > 0x7fffffffLL) return fail(Q4ADAMW_ERR_TOO_LARGE, "too many chunks for one launch");
  const SmallDesc *dev = nullptr;
  int n = 0;
  Slot *slot = nullptr;
  SmallDesc one = descs[0];
  std::unique_lock<std::mutex> lock(g_mu, std::defer_lock);
  if (descs.size() > 1) {
    lock.lock();
    void *d = nullptr;
    const int rc = stage_table(descs.data(), descs.size() * sizeof(SmallDesc), stream, &d, &slot);
    if (rc) return rc;
    dev = static_cast<const SmallDesc *>(d);
    n = (int)descs.size();
  }
  const bool pb = p_dtype == Q4ADAMW_BF16, gb = g_dtype == Q4ADAMW_BF16;
  if (!pb && !gb) launch_small(single_tensor_kernel<false, false>, chunks, stream, dev, n, one, sc);
  else if (!pb && gb) launch_small(single_tensor_kernel<false, true>, chunks, stream, dev, n, one, sc);
  else if (pb && !gb) launch_small(single_tensor_kernel<true, false>, chunks, stream, dev, n, one, sc);
  else launch_small(single_tensor_kernel<true, true>, chunks, stream, dev, n, one, sc);
  Q4_HIP(hipGetLastError());
  if (slot) return mark_slot(slot, stream);
  return 0;
}

static int check_dtypes(int p_dtype, int g_dtype) {
  if ((p_dtype != Q4ADAMW_FP32 && p_dtype != Q4ADAMW_BF16) ||
      (g_dtype != Q4ADAMW_FP32 && g_dtype != Q4ADAMW_BF16))
    return fail(Q4ADAMW_ERR_ARG, "dtype tag must be Q4ADAMW_FP32 or Q4ADAMW_BF16");
  return 0;
}

}  // namespace q4

using namespace q4;

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

int q4adamw_fused_4bit_multi(const q4adamw_tensor *tensors, int count, int p_dtype, int g_dtype,
                             float beta1, float beta2, float lr, float weight_decay, float eps,
                             float step, void *stream) {
  if (count < 0 || (count > 0 && !tensors)) return fail(Q4ADAMW_ERR_ARG, "bad tensor list");
  if (int rc = check_dtypes(p_dtype, g_dtype)) return rc;
  StepConsts sc;
  if (int rc = make_consts(beta1, beta2, lr, weight_decay, eps, step, &sc)) return rc;
  std::vector<TensorDesc> descs;
  descs.reserve(count);
  for (int i = 0; i < count; ++i) {
    const q4adamw_tensor &t = tensors[i];
    if (t.numel < 0) return fail(Q4ADAMW_ERR_ARG, "negative numel");
    if (t.numel == 0) continue;
    if (!t.p || !t.g || !t.exp_avg || !t.exp_avg_sq || !t.exp_avg_scale || !t.exp_avg_sq_scale)
      return fail(Q4ADAMW_ERR_ARG, "null tensor pointer");
    if (!aligned(t.p, 16) || !aligned(t.g, 16))
      return fail(Q4ADAMW_ERR_ALIGN, "param and grad must be 16-byte aligned");
    if (!aligned(t.exp_avg, 4) || !aligned(t.exp_avg_sq, 4) || !aligned(t.exp_avg_scale, 4) ||
        !aligned(t.exp_avg_sq_scale, 4))
      return fail(Q4ADAMW_ERR_ALIGN, "code and scale buffers must be 4-byte aligned");
    TensorDesc d;
    d.p = t.p;
    d.g = t.g;
    d.m = reinterpret_cast<uint32_t *>(t.exp_avg);
    d.v = reinterpret_cast<uint32_t *>(t.exp_avg_sq);
    d.sm = t.exp_avg_scale;
    d.sv = t.exp_avg_sq_scale;
    d.numel = t.numel;
    d.chunk0 = 0;
    descs.push_back(d);
  }
  if (descs.empty()) return 0;
  return run_fused(descs, p_dtype, g_dtype, sc, static_cast<hipStream_t>(stream));
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
  if (count < 0 || (count > 0 && !tensors)) return fail(Q4ADAMW_ERR_ARG, "bad tensor list");
  if (int rc = check_dtypes(p_dtype, g_dtype)) return rc;
  StepConsts sc;
  if (int rc = make_consts(beta1, beta2, lr, weight_decay, eps, step, &sc)) return rc;
  std::vector<SmallDesc> descs;
  descs.reserve(count);
  for (int i = 0; i < count; ++i) {
    const q4adamw_small_tensor &t = tensors[i];
    if (t.numel < 0) return fail(Q4ADAMW_ERR_ARG, "negative numel");
    if (t.numel == 0) continue;
    if (!t.p || !t.g || !t.exp_avg || !t.exp_avg_sq)
      return fail(Q4ADAMW_ERR_ARG, "null tensor pointer");
    const uintptr_t pa = p_dtype == Q4ADAMW_BF16 ? 2 : 4, ga = g_dtype == Q4ADAMW_BF16 ? 2 : 4;
    if (!aligned(t.p, pa) || !aligned(t.g, ga) || !aligned(t.exp_avg, 4) || !aligned(t.exp_avg_sq, 4))
      return fail(Q4ADAMW_ERR_ALIGN, "tensor not aligned to its element size");
    SmallDesc d;
    d.p = t.p;
    d.g = t.g;
    d.m = t.exp_avg;
    d.v = t.exp_avg_sq;
    d.numel = t.numel;
    d.chunk0 = 0;
    descs.push_back(d);
  }
  if (descs.empty()) return 0;
  return run_small(descs, p_dtype, g_dtype, sc, static_cast<hipStream_t>(stream));
}

int q4adamw_fused_single_tensor(void *p, const void *g, float *exp_avg, float *exp_avg_sq,
                                int64_t numel, int p_dtype, int g_dtype, float beta1, float beta2,
                                float lr, float weight_decay, float eps, float step,
                                void *stream) {
  q4adamw_small_tensor t = {p, g, exp_avg, exp_avg_sq, numel};
  return q4adamw_fused_single_tensor_multi(&t, 1, p_dtype, g_dtype, beta1, beta2, lr,
                                           weight_decay, eps, step, stream);
}

int q4adamw_release(void) {
  std::lock_guard<std::mutex> lock(g_mu);
  int rc = 0;
  int prev = 0;
  const bool have_prev = hipGetDevice(&prev) == hipSuccess;
  for (DevCache *c : g_caches) {
    if (hipSetDevice(c->device) != hipSuccess) continue;
    for (Slot &s : c->slots) {
      if (s.pending && s.done) (void)hipEventSynchronize(s.done);
      if (s.dev && hipFree(s.dev) != hipSuccess) rc = 1;
      if (s.host && hipHostFree(s.host) != hipSuccess) rc = 1;
      if (s.done) (void)hipEventDestroy(s.done);
    }
    delete c;
  }
  g_caches.clear();
  if (have_prev) (void)hipSetDevice(prev);
  return rc;
}

const char *q4adamw_last_error(void) { return g_err.c_str(); }

int q4adamw_version(void) { return 1000; }

}  // extern "C"
