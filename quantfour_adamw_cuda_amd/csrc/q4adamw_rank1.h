// Rank-1 scaling of the second moment, the launches around the update kernels of
// q4adamw_step.h: statistics (new second moments reduced to row and column maxima), commit,
// and the folds for tensors with several leading dimensions.
#pragma once
#include "q4adamw_device.h"

namespace q4 {

constexpr int kStatRowsPerWave = 64;     // rows a wave walks
constexpr int kStatRows = kStatRowsPerWave * kWaves;   // rows per workgroup of the statistics kernel
constexpr int kStatCols = 512;           // columns per workgroup: 8 per lane

// New second moments of a tile of kStatRows x kStatCols elements, reduced to row and
// column maxima (get_variance_tensor_statistics, adamw_fourbit_triton.py:738-746).  The
// arithmetic is the update kernel's, operation for operation, so the maxima are maxima
// of exactly the values that kernel quantizes.  The four waves of a workgroup share the
// columns and split the rows: every lane keeps 8 columns over its wave's rows, the waves'
// column maxima meet in LDS, and the tile issues one atomic per column and one per row
// (atomics on the column vector are what this kernel's time depends on most: a tile of
// 64 rows with four times as many of them took 1.25 to 2 times as long).
template <int GT, bool EXT>
__global__ __launch_bounds__(kThreads) void rank1_stats_kernel(const Rank1StatArgs args) {
  constexpr int kAhead = 4;  // rows whose loads are in flight together
  __shared__ uint32_t row_bits[4][kStatRows];       // row maxima of each 16-lane quarter of the row's wave
  __shared__ uint32_t col_bits[kWaves][kStatCols];  // column maxima of each wave
  const uint32_t chunk = args.chunk_base + blockIdx.x;
  float gscale = 1.0f;
  if (EXT && !grad_ops_begin(args.go, gscale)) return;
  const int t = find_tensor(args, chunk);
  const auto &T = args.desc[t];
  const uint32_t local = chunk - args.first_chunk[t];
  const uint32_t groups = args.col_groups[t];
  const uint32_t rg = local / groups, cg = local - rg * groups;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int64_t col = (int64_t)cg * kStatCols + lane * 8;
  const bool active = col < T.cols;  // cols is a multiple of 8: all 8 columns or none
  const int64_t tile_row0 = (int64_t)rg * kStatRows;
  const int tile_rows = (int)(tile_row0 + kStatRows < T.rows ? kStatRows : T.rows - tile_row0);
  const int wave_row0 = wave * kStatRowsPerWave;                         // within the tile
  int nrows = tile_rows - wave_row0;                                      // rows of this wave
  nrows = nrows < 0 ? 0 : (nrows > kStatRowsPerWave ? kStatRowsPerWave : nrows);
  // lanes past the last column work on zeros: code 0 under a zero scale and a zero
  // gradient give a zero second moment, which leaves every maximum alone
  float c_old[8], c_max[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    c_old[k] = active ? as_global<const float>(T.cmax)[col + k] : 0.0f;
    c_max[k] = 0.0f;
  }
  const uint32_t quarter = (uint32_t)lane >> 4;
  for (int r0 = 0; r0 < nrows; r0 += kAhead) {
    // a group past the wave's last row repeats that row: maxima do not mind
    u32x4 gw[kAhead][GT ? 1 : 2];
    uint32_t vw[kAhead];
    float r_old[kAhead];
#pragma unroll
    for (int i = 0; i < kAhead; ++i) {
      const int r = r0 + i < nrows ? r0 + i : nrows - 1;
      const int64_t row = tile_row0 + wave_row0 + r;
      r_old[i] = as_global<const float>(T.rmax)[row];
      // row bases are uniform; the lane's column is a 32-bit offset
      const int64_t row_first = row * T.cols + (int64_t)cg * kStatCols;
      const uint32_t lane_elem = (uint32_t)lane * 8u;
      const void *g_row = static_cast<const char *>(T.g) + row_first * (GT ? 2 : 4);
      const void *v_row = T.v + (row_first >> 1);
      vw[i] = 0u;
#pragma unroll
      for (int h = 0; h < (GT ? 1 : 2); ++h) gw[i][h] = u32x4{0u, 0u, 0u, 0u};
      if (active) {
        vw[i] = __builtin_amdgcn_raw_buffer_load_b32(tile_rsrc(v_row), lane_elem >> 1, 0, kNtReadOnly);
        if (GT) {
          gw[i][0] = __builtin_amdgcn_raw_buffer_load_b128(tile_rsrc(g_row), lane_elem * 2u, 0, kNtReadOnly);
        } else {
          gw[i][0] = __builtin_amdgcn_raw_buffer_load_b128(tile_rsrc(g_row), lane_elem * 4u, 0, kNtReadOnly);
          gw[i][GT ? 0 : 1] = __builtin_amdgcn_raw_buffer_load_b128(tile_rsrc(g_row), lane_elem * 4u + 16u, 0, kNtReadOnly);
        }
      }
    }
#pragma unroll
    for (int i = 0; i < kAhead; ++i) {
      float g[8];
      if constexpr (GT != 0) {
        widen_pair<GT>(gw[i][0].x, g[0], g[1]);
        widen_pair<GT>(gw[i][0].y, g[2], g[3]);
        widen_pair<GT>(gw[i][0].z, g[4], g[5]);
        widen_pair<GT>(gw[i][0].w, g[6], g[7]);
      } else {
        const u32x4 lo = gw[i][0], hi = gw[i][GT ? 0 : 1];
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
        const float v_old = code_value * min_nonneg(r_old[i], c_old[k]);
        const float v = args.b2 * v_old + args.r2 * (gk * gk);
        c_max[k] = __builtin_fmaxf(c_max[k], v);
        r_max = __builtin_fmaxf(r_max, v);
      }
      uint32_t u = f2bits(r_max);
      u = dpp_umax<0xB1>(u);
      u = dpp_umax<0x4E>(u);
      u = dpp_umax<0x141>(u);
      u = dpp_umax<0x140>(u);           // maximum of each 16-lane quarter, in all its lanes
      if ((lane & 15) == 0) row_bits[quarter][wave_row0 + r0 + i] = u;   // slots past the last row are not read
    }
  }
#pragma unroll
  for (int k = 0; k < 8; ++k) col_bits[wave][lane * 8 + k] = f2bits(c_max[k]);
  __syncthreads();
  // one atomic per column and per row of the tile
#pragma unroll
  for (int h = 0; h < kStatCols / kThreads; ++h) {
    const int c = tid + h * kThreads;
    uint32_t u = col_bits[0][c];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) u = u > col_bits[w][c] ? u : col_bits[w][c];
    const int64_t cc = (int64_t)cg * kStatCols + c;
    if (cc < T.cols && u != 0u) atomic_max_nonneg(T.cmax_next + cc, bits2f(u));
  }
#pragma unroll
  for (int h = 0; h < kStatRows / kThreads; ++h) {
    const int r = tid + h * kThreads;
    if (r < tile_rows) {
      uint32_t u = row_bits[0][r];
#pragma unroll
      for (int qi = 1; qi < 4; ++qi) u = u > row_bits[qi][r] ? u : row_bits[qi][r];
      if (u != 0u) atomic_max_nonneg(T.rmax_next + tile_row0 + r, bits2f(u));
    }
  }
}

// The same statistics for rows of any length (not a multiple of 8, or shorter than 16), where a
// row starts at any element of the packed codes: a workgroup takes kAnyStatRows rows x 256
// columns, a thread one column, element by element; the rows' maxima meet in LDS, then one
// atomic per row and per column.  Same arithmetic, operation for operation.
constexpr int kAnyStatRows = 64;
constexpr int kAnyStatCols = 256;

template <int GT, bool EXT>
__global__ __launch_bounds__(kThreads) void rank1_stats_any_kernel(const Rank1StatArgs args) {
  __shared__ uint32_t row_bits[kAnyStatRows];
  const uint32_t chunk = args.chunk_base + blockIdx.x;
  float gscale = 1.0f;
  if (EXT && !grad_ops_begin(args.go, gscale)) return;
  const int t = find_tensor(args, chunk);
  const auto &T = args.desc[t];
  const uint32_t local = chunk - args.first_chunk[t];
  const uint32_t groups = args.col_groups[t];
  const uint32_t rg = local / groups, cg = local - rg * groups;
  const int tid = threadIdx.x;
  const int64_t col = (int64_t)cg * kAnyStatCols + tid;
  const bool active = col < T.cols;
  const int64_t row0 = (int64_t)rg * kAnyStatRows;
  const int nrows = (int)(row0 + kAnyStatRows < T.rows ? kAnyStatRows : T.rows - row0);
  if (tid < kAnyStatRows) row_bits[tid] = 0u;
  __syncthreads();
  const float c_old = active ? as_global<const float>(T.cmax)[col] : 0.0f;
  float c_max = 0.0f;
  for (int r = 0; r < nrows; ++r) {
    float v = 0.0f;     // lanes past the last column leave every maximum alone
    if (active) {
      const int64_t e = (row0 + r) * T.cols + col;
      float g = load_scalar<GT>(T.g, e);
      if (EXT) g *= gscale;
      const uint32_t code = ((uint32_t)as_global<const uint8_t>(T.v)[e >> 1] >> (4 * (int)(e & 1))) & 15u;
      const float code_value = __builtin_fmaf((float)code, 0.0625f, 0.0625f);  // (code + 1) / 16, exact
      const float v_old = code_value * min_nonneg(as_global<const float>(T.rmax)[row0 + r], c_old);
      v = args.b2 * v_old + args.r2 * (g * g);
    }
    // fmaxf drops a NaN: a NaN never becomes a maximum, as in the update kernel's scales
    c_max = __builtin_fmaxf(c_max, v);
    uint32_t u = f2bits(__builtin_fmaxf(v, 0.0f));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const uint32_t o = (uint32_t)__shfl_xor((int)u, off, 64);
      u = u > o ? u : o;
    }
    if ((tid & 63) == 0 && u != 0u) atomicMax(&row_bits[r], u);
  }
  if (active && c_max != 0.0f) atomic_max_nonneg(T.cmax_next + col, c_max);
  __syncthreads();
  if (tid < nrows && row_bits[tid] != 0u) atomic_max_nonneg(T.rmax_next + row0 + tid, bits2f(row_bits[tid]));
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

// Tensors with several leading dimensions, between statistics and update: row -> its
// index in leading dimension j (row-major).
__device__ __forceinline__ int64_t lead_index(const FoldDesc &T, int64_t row, int j) {
  int64_t stride = 1;
  for (int k = T.dims - 1; k > j; --k) stride *= T.shape[k];
  return (row / stride) % T.shape[j];
}

// mode 0: every leading dimension's new statistic = maximum over the rows that share the index
// mode 1: every row's new scale = minimum over its leading statistics (after mode 0 is complete)
// mode 2: after the update, new statistics become current, their buffers return to zero
// One workgroup column per tensor (blockIdx.y), grid-stride over its rows.
template <int MODE>
__global__ __launch_bounds__(256) void rank1_fold_kernel(const FoldArgs args) {
  float gscale;
  if (!grad_ops_begin(args.go, gscale)) return;
  const FoldDesc &T = args.desc[blockIdx.y];
  const int64_t first = (int64_t)blockIdx.x * 256 + threadIdx.x, stride = (int64_t)gridDim.x * 256;
  if (MODE == 2) {
    for (int j = 0; j < T.dims; ++j) {
      for (int64_t i = first; i < T.shape[j]; i += stride) {
        as_global<float>(T.cur[j])[i] = as_global<float>(T.next[j])[i];
        as_global<float>(T.next[j])[i] = 0.0f;
      }
    }
    return;
  }
  for (int64_t row = first; row < T.rows; row += stride) {
    if (MODE == 0) {
      const float r = as_global<const float>(T.row_next)[row];
      if (r != 0.0f) {
        for (int j = 0; j < T.dims; ++j) atomic_max_nonneg(T.next[j] + lead_index(T, row, j), r);
      }
    } else {
      float s = as_global<const float>(T.next[0])[lead_index(T, row, 0)];
      for (int j = 1; j < T.dims; ++j) s = min_nonneg(s, as_global<const float>(T.next[j])[lead_index(T, row, j)]);
      as_global<float>(T.row_next)[row] = s;
    }
  }
}

}  // namespace q4
