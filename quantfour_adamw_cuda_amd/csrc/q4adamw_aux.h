// Kernels around the fused step: the non-quantized step of small tensors, the global
// gradient norm, stand-alone quantize / dequantize for checkpoint interchange.
#pragma once
#include "q4adamw_device.h"

namespace q4 {

// Non-quantized step for small tensors (cuda_adamw_kernels.cu:100-133): fp32
// moments in place, same derived scalars and operation order as the fused path.
template <int PT, int GT, bool EXT>
__global__ __launch_bounds__(256) void single_tensor_kernel(const SmallArgs args) {
  const uint32_t chunk = args.chunk_base + blockIdx.x;
  float gscale = 1.0f;
  const bool cancelled = EXT && !grad_ops_begin(args.go, gscale);
  const bool zero_g = EXT && args.go.zero != 0u;
  if (cancelled && !zero_g) return;
  const int t = find_tensor(args, chunk);
  const SmallDesc &T = args.desc[t];
  const StepConsts sc = EXT ? step_consts(args.sc, args.go) : args.sc;
  const int64_t base = (int64_t)(chunk - args.first_chunk[t]) * kSmallChunk;
  const int64_t end = base + kSmallChunk < T.numel ? base + kSmallChunk : T.numel;
  if (cancelled) {  // a cancelled step still clears the gradients it was asked to clear
    for (int64_t i = base + threadIdx.x; i < end; i += 256) {
      store_scalar<GT>(const_cast<void *>(T.g), i, 0.0f);
    }
    return;
  }
  for (int64_t i = base + threadIdx.x; i < end; i += 256) {
    float gi = load_scalar<GT>(T.g, i);
    if (EXT) {
      gi *= gscale;
      if (zero_g) {
        store_scalar<GT>(const_cast<void *>(T.g), i, 0.0f);
      }
    }
    const float pi = load_scalar<PT>(T.p, i);
    const float m = sc.b1 * as_global<const float>(T.m)[i] + sc.r1 * gi;
    const float v = sc.b2 * as_global<const float>(T.v)[i] + sc.r2 * (gi * gi);
    as_global<float>(T.m)[i] = m;
    as_global<float>(T.v)[i] = v;
    // exact form here: these tensors are tiny, so the divisions cost nothing
    const float den = __builtin_sqrtf(v) / sc.c2s + sc.eps;
    const float pn = pi * sc.wdu - sc.ss * (m / den);
    store_scalar<PT>(T.p, i, pn);
  }
}


// ---------------------------------------------------------------------------
// a step whose number lives on the device
// ---------------------------------------------------------------------------
// One thread: advances the step counter and derives the step's scalars exactly as the
// host does for a step it knows (make_consts; optim/cuda_adamw_kernels.cu:435-440), from
// the bias-correction pair the host tabulated for that step number: every operation
// below is the IEEE operation the host performs, so the scalars agree bit for bit.  A
// set overflow flag leaves counter and scalars alone (the step's launches do nothing then).
__global__ void device_step_kernel(float *counter_, const float *table_, int64_t first_step, int64_t table_steps,
                                   const float *lr_dev, float beta1, float beta2, float lr, float wd, float eps,
                                   const float *skip, StepConsts *out_) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  if (skip && *as_global<const float>(skip) != 0.0f) return;
  const gptr<float> counter = as_global<float>(counter_);
  const float t = *counter + 1.0f;
  *counter = t;
  int64_t k = (int64_t)t - first_step;
  k = k < 0 ? 0 : (k >= table_steps ? table_steps - 1 : k);   // past the table: its last, converged entry
  const float c1 = as_global<const float>(table_)[2 * k], c2s = as_global<const float>(table_)[2 * k + 1];
  const float lrv = lr_dev ? *as_global<const float>(lr_dev) : lr;
  StepConsts sc;
  sc.b1 = beta1;
  sc.b2 = beta2;
  sc.r1 = 1.0f - beta1;
  sc.r2 = 1.0f - beta2;
  const float lrwd = lrv * wd;
  sc.wdu = 1.0f - lrwd;
  sc.ss = lrv / c1;
  sc.c2s = c2s;
  sc.eps = eps;
  const double den_scale = 1.0 / ((double)c2s * (double)sc.ss), den_eps = (double)eps / (double)sc.ss;
  const bool fits = den_scale <= (double)FLT_MAX && den_eps <= (double)FLT_MAX;
  sc.den_scale = fits ? (float)den_scale : 0.0f;
  sc.den_eps = fits ? (float)den_eps : __builtin_inff();
  const gptr<float> o = as_global<float>(out_);   // the order step_consts() reads
  o[0] = sc.b1; o[1] = sc.b2; o[2] = sc.r1; o[3] = sc.r2; o[4] = sc.wdu;
  o[5] = sc.ss; o[6] = sc.c2s; o[7] = sc.eps; o[8] = sc.den_scale; o[9] = sc.den_eps;
  as_global<uint32_t>(out_)[10] = (uint32_t)t;   // the step number, for the rounding noise's salt
  make_exact_consts(&sc);
  o[11] = sc.c2s_rcp;
  as_global<uint32_t>(out_)[12] = sc.exact_short;
}

// ---------------------------------------------------------------------------
// self-check of the exact parameter update's short forms on the running GPU
// ---------------------------------------------------------------------------
// Walks every fp32 pattern of the short forms' domains through them and counts disagreements
// with the correctly rounded results, taken in fp64 and rounded to fp32 (for a square root, a
// reciprocal and a quotient the second rounding is harmless: 53 >= 2 * 24 + 2 bits):
//   out[0]  sqrt_rn(x) != RN(sqrt x)                      x in [2^-96, 2^90]
//   out[1]  estimate + one Newton step != RN(1 / d)       d in [2^-60, 2^60]
//   out[2]  div_rn(m, d) != RN(m / d)                     every such d with three numerators:
//           1, and two of either sign with a mantissa and exponent (2^-60 .. 2^59) hashed from d
//   out[3]  the compiler's general sqrtf != RN(sqrt x)    (what lanes outside the domains take)
//   out[4]  the compiler's general m / d != RN(m / d)
//   out[5]  patterns walked
// out[1] is a property of the hardware's reciprocal estimate: arithmetic alone promises it only
// for divisors whose mantissa is not all ones.
__global__ __launch_bounds__(256) void rounding_selfcheck_kernel(unsigned long long *out_) {
  const gptr<unsigned long long> out = as_global<unsigned long long>(out_);
  unsigned long long bad[5] = {0, 0, 0, 0, 0}, walked = 0;
  const uint32_t first = (blockIdx.x * 256u + threadIdx.x) << 11;   // 2^21 threads x 2^11 patterns = 2^32
  for (uint32_t k = 0; k < 2048u; ++k) {
    const uint32_t u = first + k;
    const float x = bits2f(u);
    if (x >= kExactVLo && x <= kExactVHi) {
      const float want = (float)__builtin_sqrt((double)x);
      bad[0] += f2bits(sqrt_rn(x)) != f2bits(want);
      bad[3] += f2bits(__builtin_sqrtf(x)) != f2bits(want);
      ++walked;
    }
    if (x >= kExactLo && x <= kExactHi) {
      const float y0 = __builtin_amdgcn_rcpf(x);
      const float y = __builtin_fmaf(__builtin_fmaf(-x, y0, 1.0f), y0, y0);
      bad[1] += f2bits(y) != f2bits((float)(1.0 / (double)x));
      const uint32_t h = lowbias32(u);
      const float m1 = bits2f((h & 0x807fffffu) | ((67u + (h >> 23) % 120u) << 23));
      const float ms[3] = {1.0f, m1, -m1 * 0.75f};
#pragma unroll
      for (int j = 0; j < 3; ++j) {
        const float want = (float)((double)ms[j] / (double)x);
        bad[2] += f2bits(div_rn(ms[j], x)) != f2bits(want);
        bad[4] += f2bits(ms[j] / x) != f2bits(want);
      }
      ++walked;
    }
  }
#pragma unroll
  for (int j = 0; j < 5; ++j) {
    if (bad[j]) atomicAdd(out_ + j, bad[j]);
  }
  atomicAdd(out_ + 5, walked);
  (void)out;
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
template <int GT>
__global__ __launch_bounds__(256) void grad_sumsq_kernel(const NormArgs args) {
  constexpr int kElemBytes = GT ? 2 : 4;
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
          if constexpr (GT != 0) {
            float lo, hi;
            widen_pair<GT>(u[c], lo, hi);
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
        const double x = (double)load_scalar<GT>(cb, i);
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
                                                       float *__restrict__ scale_, int64_t group0) {
  const gptr<const float> x = as_global<const float>(x_);
  const int lane = threadIdx.x & 63;
  const int64_t blk = (group0 + blockIdx.x) * 4 + (threadIdx.x >> 6);   // group0: this grid's first workgroup
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
// 15-compare count (optim/adamw_fourbit_triton.py:834-863).  Rows may have any length, so the
// byte's two elements find their rows and columns separately.
__global__ __launch_bounds__(256) void quantize_rank1_kernel(const float *x_, int64_t rows, int64_t cols,
                                                             const float *row_max, const float *col_max,
                                                             uint8_t *codes_, int64_t group0) {
  const int64_t e = ((group0 + blockIdx.x) * 256 + threadIdx.x) * 2;
  const int64_t numel = rows * cols;
  if (e >= numel) return;
  uint32_t byte = 0;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    if (e + h >= numel) break;     // an odd element count: the last byte's high nibble stays 0
    const int64_t i = (e + h) / cols, j = (e + h) - i * cols;
    const float q = as_global<const float>(x_)[e + h] /
                    __builtin_fminf(as_global<const float>(row_max)[i], as_global<const float>(col_max)[j]);
#pragma unroll
    for (int k = 0; k < 15; ++k) byte += (qmid_v(k) < q) ? (1u << (4 * h)) : 0u;
  }
  as_global<uint8_t>(codes_)[e >> 1] = (uint8_t)byte;
}

// optim/adamw_fourbit_triton.py:520-527: code-book entry times min(row, column maximum)
__global__ __launch_bounds__(256) void dequantize_rank1_kernel(const uint8_t *codes_, const float *row_max,
                                                               const float *col_max, int64_t rows,
                                                               int64_t cols, float *out_, int64_t group0) {
  const int64_t e = ((group0 + blockIdx.x) * 256 + threadIdx.x) * 2;
  const int64_t numel = rows * cols;
  if (e >= numel) return;
  const uint32_t byte = as_global<const uint8_t>(codes_)[e >> 1];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    if (e + h >= numel) break;
    const int64_t i = (e + h) / cols, j = (e + h) - i * cols;
    as_global<float>(out_)[e + h] = qmap_v((int)((byte >> (4 * h)) & 15u)) *
                                    __builtin_fminf(as_global<const float>(row_max)[i], as_global<const float>(col_max)[j]);
  }
}

// cuda_adamw_kernels.cu:329-343: code -> code-book entry * block scale
template <bool SECOND>
__global__ __launch_bounds__(256) void dequantize_kernel(const uint8_t *__restrict__ codes_,
                                                         const float *__restrict__ scale_,
                                                         int64_t numel, float *__restrict__ out_, int64_t group0) {
  const int64_t e = ((group0 + blockIdx.x) * 256 + threadIdx.x) * 2;
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

}  // namespace q4
