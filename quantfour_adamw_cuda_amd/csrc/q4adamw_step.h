// The fused 4-bit AdamW step: one tile of one tensor (process_tile) and the kernels built on
// it -- block-scaled, and the update kernels of the rank-1 scaled second moment -- each with
// nearest or stochastic rounding, with or without gradient options, and with the folded or
// the exact form of the parameter update.
#pragma once
#include "q4adamw_device.h"

namespace q4 {

// Geometry of the fused kernel: a lane owns 16 bytes of the widest of the parameter and
// gradient streams, so that no stream needs two accesses per lane.
template <int PT, int GT>
struct Geometry {
  static constexpr int kEpl = (PT && GT) ? 8 : 4;      // elements per lane
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
// EXACT: the parameter comes from the reference's expression with each of its seven
// operations rounded as IEEE 754 rounds it (optim/cuda_adamw_kernels.cu:334,351), by short
// sequences inside their domains and the general expansions outside them; otherwise from the
// folded form with the hardware's square root and reciprocal (a tolerance).
// SHAPE (with RANK1): how a tile lies in its matrix.  kTileWide: rows are at least a tile
// long, so a tile touches one row or two.  kTileNarrow: rows may be shorter than a tile.
// kTileRows: rows are a whole number of quantization blocks long and tiles start at the
// beginning of a row, so that the workgroup's four waves work on the same columns of four
// consecutive rows: they fetch the columns' maxima once, together, and pass them through LDS
// (RowsTile).  kTileRowsLast is the same for the last tile of a row that is not a whole
// number of tiles long: its first RowsTile::width elements are there (whole blocks), the
// lanes of the others load nothing, work on zeros and store nothing.  kTileAny: rows of any
// length (not a multiple of 8, or shorter than 16): every element finds its own row and column
// (matrices of fewer than 2^32 elements).
constexpr int kTileWide = 0, kTileNarrow = 1, kTileRows = 2, kTileRowsLast = 3, kTileAny = 4;

// What a wave of the kTileRows form knows beyond its tile number: its row, the tile's first
// column, and this thread's share of the workgroup's fetch of the columns' maxima (old and
// new; kTile / 256 consecutive columns per thread), which goes to `columns` in LDS:
// [0, kTile) old, [kTile, 2 kTile) 16 / max(new, kScaleLo) -- the reciprocal every element of
// the column would otherwise take for itself -- and [2 kTile, 3 kTile) new, which only the
// exact path reads.
struct RowsTile {
  int64_t row;
  uint32_t col0;
  uint32_t width;     // elements of the tile that lie in the row: kTile, or less in a row's last tile
  float *columns;
  float2 share_old, share_new;
};

// Writes a thread's share of the columns' maxima into LDS (before the workgroup's barrier).
template <int N>
__device__ __forceinline__ void stage_columns(const RowsTile &rt, int tid) {
  const float inv_x = __builtin_amdgcn_rcpf(max_nonneg(rt.share_new.x, kScaleLo)) * 16.0f;
  if (N == 4) {
    rt.columns[tid] = rt.share_old.x;
    rt.columns[64 * N + tid] = inv_x;
    rt.columns[128 * N + tid] = rt.share_new.x;
  } else {
    const float inv_y = __builtin_amdgcn_rcpf(max_nonneg(rt.share_new.y, kScaleLo)) * 16.0f;
    *reinterpret_cast<float2 *>(rt.columns + 2 * tid) = rt.share_old;
    *reinterpret_cast<float2 *>(rt.columns + 64 * N + 2 * tid) = make_float2(inv_x, inv_y);
    *reinterpret_cast<float2 *>(rt.columns + 128 * N + 2 * tid) = rt.share_new;
  }
}

template <int PT, int GT, bool FULL, bool EXT, bool RANK1, bool SR, int SHAPE, bool EXACT, typename Desc>
__device__ __forceinline__ void process_tile(const Desc &T, int64_t tb, int lane, int wave, int tid,
                                             const StepConsts &sc, uint2 *lds, const TableSlot &slot,
                                             float gscale, bool zero_g, uint32_t salt,
                                             const RowsTile *rt = nullptr) {
  using G = Geometry<PT, GT>;
  constexpr int N = G::kEpl;
  constexpr bool kRows = SHAPE == kTileRows || SHAPE == kTileRowsLast;
  // Uniform (scalar) part of every address: the tile's first element tb (a multiple of the
  // block size), its byte and block; the per-lane part is a small 32-bit offset.
  const int64_t numel = T.numel;
  const void *p_tile = static_cast<const char *>(T.p) + tb * (PT ? 2 : 4);
  const void *g_tile = static_cast<const char *>(T.g) + tb * (GT ? 2 : 4);
  const uint8_t *m_tile = T.m + (tb >> 1);
  const uint8_t *v_tile = T.v + (tb >> 1);
  const float *sm_tile = T.sm + tb / Q4ADAMW_BLOCK;
  const float *sv_tile = nullptr;
  if constexpr (!RANK1) sv_tile = T.sv + tb / Q4ADAMW_BLOCK;
  const uint32_t e0 = (uint32_t)lane * N;                          // first element of this lane in the tile
  bool lane_on = true;                                             // whether the lane's elements exist
  if constexpr (SHAPE == kTileRowsLast) lane_on = e0 < rt->width;
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
  Vals<N> ro, rn;   // kTileAny: the row maxima of every element
  if constexpr (RANK1 && SHAPE == kTileAny) {
    // T.div_magic / div_shift divide by cols; indices of elements past the end are clamped
    const uint32_t first = (uint32_t)tb + e0, cols = (uint32_t)T.cols, last = (uint32_t)T.rows - 1u;
#pragma unroll
    for (int j = 0; j < N; ++j) {
      const uint32_t e = first + (uint32_t)j;
      uint32_t row = fast_div(e, T.div_magic, T.div_shift);
      const uint32_t col = e - row * cols;
      row = row < last ? row : last;
      ro.x[j] = as_global<const float>(T.rmax)[row];
      rn.x[j] = as_global<const float>(T.rmax_next)[row];
      c_old.x[j] = as_global<const float>(T.cmax)[col];
      c_new.x[j] = as_global<const float>(T.cmax_next)[col];
    }
  } else if constexpr (RANK1) {
    // (row, column) of the tile's first element, in units of 8 elements so that the
    // division is a 32-bit one.  A lane's N elements (N = 4 or 8, first one a multiple of N)
    // lie in one row, because rows are multiples of 8 elements long.
    const uint32_t tb8 = (uint32_t)(tb >> 3), cols8 = (uint32_t)(T.cols >> 3);  // numel < 2^35
    const int64_t last = T.rows - 1;
    uint32_t col;
    if constexpr (kRows) {
      // the whole tile lies in one row; the columns' maxima come through LDS further down
      col = rt->col0 + e0;
      // the statistics are complete before this kernel starts and change after it ends
      r_old = as_constant<const float>(T.rmax)[rt->row];
      r_new = as_constant<const float>(T.rmax_next)[rt->row];
    } else if constexpr (SHAPE == kTileWide) {
      // a tile is no longer than a row, so a lane is in the tile's first row or in the next
      const uint32_t row32 = fast_div(tb8, T.div_magic, T.div_shift);
      const int64_t row = row32;
      const uint32_t col0 = (tb8 - row32 * cols8) << 3;
      col = col0 + e0;
      const bool wrapped = col >= (uint32_t)T.cols;
      if (wrapped) col -= (uint32_t)T.cols;
      const int64_t ra = row < last ? row : last, rb = row + 1 < last ? row + 1 : last;  // past-the-end lanes stay in bounds
      const float r_old_a = as_global<const float>(T.rmax)[ra], r_old_b = as_global<const float>(T.rmax)[rb];
      const float r_new_a = as_global<const float>(T.rmax_next)[ra], r_new_b = as_global<const float>(T.rmax_next)[rb];
      r_old = wrapped ? r_old_b : r_old_a;
      r_new = wrapped ? r_new_b : r_new_a;
    } else {
      // a tile may span several rows (the matrix is narrower than a tile): every lane finds its own
      const uint32_t u8 = tb8 + (e0 >> 3);
      const uint32_t row32 = fast_div(u8, T.div_magic, T.div_shift);
      col = ((u8 - row32 * cols8) << 3) + (e0 & 7u);
      const int64_t row = (int64_t)row32 < last ? (int64_t)row32 : last;   // past-the-end lanes stay in bounds
      r_old = as_global<const float>(T.rmax)[row];
      r_new = as_global<const float>(T.rmax_next)[row];
    }
    if constexpr (!kRows) {
#pragma unroll
      for (int k = 0; k < N; k += 4) {
        const u32x4 a = __builtin_amdgcn_raw_buffer_load_b128(tile_rsrc(T.cmax), (col + k) * 4u, 0, 0);
        const u32x4 b = __builtin_amdgcn_raw_buffer_load_b128(tile_rsrc(T.cmax_next), (col + k) * 4u, 0, 0);
        c_old.x[k] = bits2f(a.x); c_old.x[k + 1] = bits2f(a.y); c_old.x[k + 2] = bits2f(a.z); c_old.x[k + 3] = bits2f(a.w);
        c_new.x[k] = bits2f(b.x); c_new.x[k + 1] = bits2f(b.y); c_new.x[k + 2] = bits2f(b.z); c_new.x[k + 3] = bits2f(b.w);
      }
    }
  }

  float p[N], g[N];
  if constexpr (SHAPE == kTileRowsLast) {
#pragma unroll
    for (int j = 0; j < N; ++j) p[j] = g[j] = 0.0f;
  }
  if (lane_on) {
    load_elems<PT, N, FULL>(p_tile, e0, nv, p);
    load_elems<GT, N, FULL>(g_tile, e0, nv, g);
  }
  if (EXT) {
#pragma unroll
    for (int j = 0; j < N; ++j) g[j] *= gscale;
    if (zero_g && lane_on) zero_elems<GT, N, FULL>(const_cast<void *>(g_tile), e0, nv);
  }
  uint32_t mw = 0, vw = 0;
  if (!lane_on) {
    // nothing to read: zero codes under a zero scale
  } else if (FULL) {
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
  if (!lane_on) {
  } else if (FULL) {
    // scales are 4 bytes per block: cached, so that neighbouring blocks share lines
    sm_old = bits2f(__builtin_amdgcn_raw_buffer_load_b32(tile_rsrc(sm_tile), blk * 4u, 0, 0));
    if (!RANK1) sv_old = bits2f(__builtin_amdgcn_raw_buffer_load_b32(tile_rsrc(sv_tile), blk * 4u, 0, 0));
  } else if (blk_ok) {
    sm_old = as_global<const float>(sm_tile)[blk];
    if (!RANK1) sv_old = as_global<const float>(sv_tile)[blk];
  }
  // this block's dequantization tables: entry i = beta1 * (code_book_m[i] * scale_m) of the
  // first moment's, beta2 * (code_book_v[i] * scale_v) of the second moment's: the old
  // moments (cuda_adamw_kernels.cu:340,343) with the first product of their updates
  // (:341,344) already applied, each product rounded as the per-element form rounds it.
  // Written by the block's lanes (lane & 15 = i) into the wave's private LDS regions.  Two
  // tables of 4-byte entries, not one of pairs: a block's 16 entries then lie in 16
  // different banks and neighbouring blocks in the other 16, so that a wave's reads, with
  // every lane choosing its own entry, do not collide (pairs left half the banks idle in
  // every read).  Rank-1: the second entry is the bare code-book value; scale and beta2
  // follow per element.
  char *lds_bytes = reinterpret_cast<char *>(lds);
  const uint32_t cb_entry = (uint32_t)wave * 64u + blk * 16u;  // entry number of code 0
  {
    const float m_entry = sc.b1 * (slot.qm * sm_old);
    const float v_entry = RANK1 ? qmap_v(lane & 15) : sc.b2 * (qmap_v(lane & 15) * sv_old);
    float *entry = reinterpret_cast<float *>(lds_bytes) + cb_entry + ((uint32_t)lane & 15u);
    entry[0] = m_entry;
    entry[kLdsSecondMoment] = v_entry;
  }
  if constexpr (RANK1 && kRows) stage_columns<N>(*rt, tid);
  setup_tables<SR>(lds, tid, slot);
  if constexpr (RANK1 && kRows) {
#pragma unroll
    for (int k = 0; k < N; k += 4) {
      // c_new: 16 / max(new column maximum, kScaleLo) in this form, not the maximum itself
      const float4 a = *reinterpret_cast<const float4 *>(rt->columns + e0 + k);
      const float4 b = *reinterpret_cast<const float4 *>(rt->columns + 64 * N + e0 + k);
      c_old.x[k] = a.x; c_old.x[k + 1] = a.y; c_old.x[k + 2] = a.z; c_old.x[k + 3] = a.w;
      c_new.x[k] = b.x; c_new.x[k + 1] = b.y; c_new.x[k + 2] = b.z; c_new.x[k + 3] = b.w;
    }
  }

  // entry numbers of the lane's codes, one per byte: even elements, odd elements
  const uint32_t three = 3u, two = 2u;
  const uint32_t cb_bytes = __builtin_amdgcn_perm(cb_entry, cb_entry, 0u);   // the entry number (< 256) in all four bytes
  const uint32_t m_even = and_or(mw, 0x0F0F0F0Fu, cb_bytes), m_odd = and_or(mw >> 4, 0x0F0F0F0Fu, cb_bytes);
  const uint32_t v_even = and_or(vw, 0x0F0F0F0Fu, cb_bytes), v_odd = and_or(vw >> 4, 0x0F0F0F0Fu, cb_bytes);

  // dequantize, update moments and parameter (cuda_adamw_kernels.cu:334-351)
  Vals<N> mn, vn;
  float am = 0.0f, av = 0.0f;
  float m_least = kExactHi, v_least = kExactVHi;   // EXACT: the lane's smallest |m| and v
  float p_new[N];
#pragma unroll
  for (int j = 0; j < N; ++j) {
    const uint32_t mo = entry_offset(j & 1 ? m_odd : m_even, j >> 1, two);
    const uint32_t vo = entry_offset(j & 1 ? v_odd : v_even, j >> 1, two);
    const float m_old = *reinterpret_cast<const float *>(lds_bytes + mo);
    float v_old = *reinterpret_cast<const float *>(lds_bytes + vo + kLdsSecondMoment * 4u);
    if constexpr (RANK1) v_old = sc.b2 * (v_old * min_nonneg(SHAPE == kTileAny ? ro.x[j] : r_old, c_old.x[j]));  // adamw_fourbit_triton.py:520-527
    const float gj = g[j];
    float m = m_old + sc.r1 * gj;                 // m_old, v_old: beta times the old moment
    float v = v_old + sc.r2 * (gj * gj);
    if (!FULL && j >= nv) { m = 0.0f; v = 0.0f; }
    if constexpr (EXACT) {
      // the reference's seven operations, each rounded as IEEE 754 rounds it
      // (cuda_adamw_kernels.cu:334,351), valid inside the ranges checked below
      const float den = div_by_reciprocal(sqrt_rn(v), sc.c2s, sc.c2s_rcp) + sc.eps;
      p_new[j] = p[j] * sc.wdu - sc.ss * div_rn(m, den);
      m_least = __builtin_fminf(m_least, __builtin_fabsf(m));
      v_least = __builtin_fminf(v_least, v);
    } else {
      // folded form: the hardware's 1-ulp square root and a reciprocal in place of the
      // divisions; the parameters then agree with the reference's to a tolerance only
      const float den = __builtin_fmaf(__builtin_amdgcn_sqrtf(v), sc.den_scale, sc.den_eps);
      p_new[j] = __builtin_fmaf(-m, __builtin_amdgcn_rcpf(den), p[j] * sc.wdu);
    }
    mn.x[j] = m;
    vn.x[j] = v;
    am = __builtin_fmaxf(am, __builtin_fabsf(m));
    av = __builtin_fmaxf(av, v);
  }
  if constexpr (EXACT) {
    // The short forms hold for moments inside [2^-60, 2^60] and [2^-96, 2^90] and for step
    // constants that keep the denominator inside [2^-60, 2^60]; a NaN moment passes (the
    // minima and maxima skip it) and comes out as the NaN the reference produces.  Any other
    // lane -- zeros among them -- takes the general expansions for its elements.
    const bool in_range = m_least >= kExactLo && am <= kExactHi && v_least >= kExactVLo && av <= kExactVHi;
    if (__builtin_expect(!(sc.exact_short != 0u && in_range), 0)) {
#pragma unroll
      for (int j = 0; j < N; ++j) p_new[j] = param_update_ieee(p[j], mn.x[j], vn.x[j], sc);
    }
  }
  if (lane_on) store_elems<PT, N, FULL>(const_cast<void *>(p_tile), e0, nv, p_new);

  // block scales (exact: max is order independent)
  const float v_lane_max = av;
  if (G::kLanesPerBlock == 32) {
    block_max32_pair(am, av);
  } else {
    am = row_max16(am);
    if (!RANK1) av = row_max16(av);
  }
  if (blk_ok && lane_on && (lane & (G::kLanesPerBlock - 1)) == 0) {
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
  // smallest fractional part of a code coordinate shifted up by the guard band: second
  // moment 16 q - 1/2 (nearest), both moments' coordinate minus noise (stochastic)
  float vfrac = 1.0f;
  // rank-1: the new scale of every element and 16 / scale.  The hardware reciprocal's
  // one ulp is well inside the second moment's guard band (2^-17 in units of 16 q), so
  // it goes unrefined.  Scales below the safe range are clamped for the reciprocal: a
  // zero value under a zero scale then still gets code 0; any other value under such a
  // scale sends the lane to the exact path.
  Vals<N> s_new, inv16;
  if constexpr (RANK1 && kRows) {
    // 16 / min(row maximum, column maximum) is the larger of the two reciprocals, the row's
    // taken once per lane and the columns' once per workgroup (stage_columns): one
    // instruction per element.  (Where the hardware reciprocal is not monotonic the other
    // one is within an ulp of it, which the guard band covers all the same.)  A clamped
    // scale shows as the reciprocal of the clamp.
    const float row_inv16 = __builtin_amdgcn_rcpf(max_nonneg(r_new, kScaleLo)) * 16.0f;
    float inv_max = 0.0f;
#pragma unroll
    for (int j = 0; j < N; ++j) {
      inv16.x[j] = max_nonneg(row_inv16, c_new.x[j]);
      inv_max = max_nonneg(inv_max, inv16.x[j]);
    }
    redo |= r_new > kScaleHi || (inv_max >= kInvScaleLo16 && v_lane_max != 0.0f);
  } else if constexpr (RANK1 && SHAPE == kTileAny) {
    float s_least = rn.x[0], s_most = 0.0f;
#pragma unroll
    for (int j = 0; j < N; ++j) {
      const float sj = min_nonneg(rn.x[j], c_new.x[j]);      // adamw_fourbit_triton.py:749-755
      s_new.x[j] = sj;
      s_least = min_nonneg(s_least, sj);
      s_most = max_nonneg(s_most, sj);
      inv16.x[j] = __builtin_amdgcn_rcpf(max_nonneg(sj, kScaleLo)) * 16.0f;
    }
    redo |= s_most > kScaleHi || (s_least < kScaleLo && v_lane_max != 0.0f);
  } else if constexpr (RANK1) {
    float c_min = c_new.x[0];
#pragma unroll
    for (int j = 0; j < N; ++j) {
      const float sj = min_nonneg(r_new, c_new.x[j]);        // adamw_fourbit_triton.py:749-755
      s_new.x[j] = sj;
      c_min = min_nonneg(c_min, c_new.x[j]);
      inv16.x[j] = __builtin_amdgcn_rcpf(max_nonneg(sj, kScaleLo)) * 16.0f;
    }
    // every scale is at most r_new and at least min(r_new, c_min)
    redo |= r_new > kScaleHi || (min_nonneg(r_new, c_min) < kScaleLo && v_lane_max != 0.0f);
  }
  uint32_t mword = 0, vword = 0;
  // stochastic rounding: the elements' 16-bit noise numbers n as floats; the noise itself is
  // (2 n + 1) / 2^17 = n * kNoiseStep + kVGuard, and the fast path works with code
  // coordinates shifted up by the guard band, so the two halves of a step cancel there
  Vals<N> um, uv;
  if constexpr (SR) {
    // key = low half of the element index, xor the salt, xor the mixed high half
    const uint32_t tile_salt = salt ^ ((uint32_t)((uint64_t)tb >> 32) * 0x9E3779B9u);
    // a tile never straddles a multiple of 2^32 (the launcher sees to it: tiles start at
    // multiples of their length, or the matrix is small enough, rank1_shape); the lane's first
    // element is a multiple of N, so element j's key is the first one's with j in its low bits
    const uint32_t key0 = ((uint32_t)tb + e0) ^ tile_salt;
#pragma unroll
    for (int j = 0; j < N; ++j) {
      const uint32_t y = lowbias32_open(key0 ^ (uint32_t)j);   // the hash is y ^ (y >> 16)
      um.x[j] = hash_high_half_as_float(y);
      uv.x[j] = hash_low_half_as_float(y);
    }
  }
#pragma unroll
  for (int j = 0; j < N; j += 2) {
    // first moment: the quotients' bucket entries, two quotients per conversion
    const float q0 = mn.x[j] * rm, q1 = mn.x[j + 1] * rm;
    const uint32_t halves = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(q0, q1));
    const uint2 ent0 = *reinterpret_cast<const uint2 *>(lds_bytes + kLdsBuckets * 8u + byte_shifted<1>(halves, three));
    const uint2 ent1 = *reinterpret_cast<const uint2 *>(lds_bytes + kLdsBuckets * 8u + byte_shifted<3>(halves, three));
    if constexpr (SR) {
      // interval among the code-book entries; inside it the code is floor(k + position -
      // noise), an affine function of the quotient.  Computed shifted up by the guard band
      // (coordinate - n * kNoiseStep): a fractional part below twice the band then marks a
      // value within the band of an integer on either side, which goes to the exact path,
      // and every other value truncates to its code.  Error budget in units of one code: the
      // quotient is within 2^-22 relative of the exact one and |q| / width < 9 (2.25 *
      // 2^-20), the map's two roundings and the two operations here add 2^-21 each: 0.54 of
      // the band.  The value is never negative, and below 16 outside the band.
      const float qq[2] = {q0, q1};
      const uint2 ent[2] = {ent0, ent1};
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const uint32_t interval = high_half_if_ge(qq[h], bits2f(ent[h].x), ent[h].y);   // byte offset into the affine table
        const float2 af = *reinterpret_cast<const float2 *>(lds_bytes + kLdsIntervals * 8u + interval);
        const float y = __builtin_fmaf(um.x[j + h], -kNoiseStep, __builtin_fmaf(qq[h], af.x, af.y));
        vfrac = __builtin_fminf(vfrac, __builtin_amdgcn_fractf(y));
        mword = append_code<N>(mword, (uint32_t)(int)y, j + h);
      }
    } else {
      const bool hi0 = q0 > bits2f(ent0.y), hi1 = q1 > bits2f(ent1.y);
      redo |= hi0 != (q0 > bits2f(ent0.x));
      redo |= hi1 != (q1 > bits2f(ent1.x));
      // base code in the entry's low nibble, plus one above the threshold; every
      // code enters the word at the top and moves down four bits per later element
      mword = __builtin_amdgcn_alignbit(ent0.x + (hi0 ? 1u : 0u), mword, 4);
      mword = __builtin_amdgcn_alignbit(ent1.x + (hi1 ? 1u : 0u), mword, 4);
    }

    // second moment: thresholds at 16q = k + 0.5, k = 1..15
#pragma unroll
    for (int k = j; k < j + 2; ++k) {
      if constexpr (SR) {
        // code-book entries at 16 q = 1..16: interval number floor(16 q), position in it
        // fract(16 q), up iff noise < position, i.e. code = floor(16 q - noise) wherever
        // that difference is clear of an integer; shifted up by the guard band as for the
        // first moment.  The shifted value is above -1 (truncation gives 0 below 0) and,
        // outside the band, below 16.
        const float y = __builtin_fmaf(vn.x[k], RANK1 ? inv16.x[k] : rv16, uv.x[k] * -kNoiseStep);
        vfrac = __builtin_fminf(vfrac, __builtin_amdgcn_fractf(y));
        vword = append_code<N>(vword, (uint32_t)(int)y, k);
      } else {
        const float t = __builtin_fmaf(vn.x[k], RANK1 ? inv16.x[k] : rv16, kVGuard - 0.5f);
        vfrac = __builtin_fminf(vfrac, __builtin_amdgcn_fractf(t));
        // t > -1, so truncation gives 0 for t < 0
        vword = append_code<N>(vword, (uint32_t)(int)t, k);
      }
    }
  }
  if (N == 4 && !SR) mword >>= 16;   // four codes entered at the top
  redo |= vfrac < 2.0f * kVGuard;
  if (__builtin_expect(redo, 0)) {
    if constexpr (RANK1 && kRows) {
      // the scales themselves: the new column maxima are the third array of the staging area
#pragma unroll
      for (int k = 0; k < N; k += 4) {
        const float4 c = *reinterpret_cast<const float4 *>(rt->columns + 128 * N + e0 + k);
        s_new.x[k] = min_nonneg(r_new, c.x);                  // adamw_fourbit_triton.py:749-755
        s_new.x[k + 1] = min_nonneg(r_new, c.y);
        s_new.x[k + 2] = min_nonneg(r_new, c.z);
        s_new.x[k + 3] = min_nonneg(r_new, c.w);
      }
    }
    if constexpr (SR) {
#pragma unroll
      for (int j = 0; j < N; ++j) {
        um.x[j] = sr_noise_value(um.x[j]);
        uv.x[j] = sr_noise_value(uv.x[j]);
      }
      mword = quantize_exact_sr<false, N>(mn, am, um);
      if constexpr (RANK1) vword = quantize_exact_sr_scales<N>(vn, s_new, uv);
      else vword = quantize_exact_sr<true, N>(vn, av, uv);
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

  if (!lane_on) {
  } else if (FULL) {
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

template <int PT, int GT, bool EXT, bool SR, bool EXACT>
__global__ __launch_bounds__(kThreads) void fused_4bit_kernel(const FusedArgs args) {
  using G = Geometry<PT, GT>;
  __shared__ uint2 lds[kLdsEntries];
  const int tid = threadIdx.x;
  const TableSlot slot = request_table_slot<SR>(tid);
  const uint32_t chunk = args.chunk_base + (blockIdx.x & 7u) * args.chunks_per_xcd + (blockIdx.x >> 3);
  if (chunk >= args.nchunks) return;  // whole workgroup: the grid is padded to a multiple of 8
  float gscale = 1.0f;
  const bool cancelled = EXT && !grad_ops_begin(args.go, gscale);  // whole grid
  const bool zero_g = EXT && args.go.zero != 0u;
  if (cancelled && !zero_g) return;
  const int t = find_tensor(args, chunk);
  const TensorDesc &T = args.desc[t];
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int64_t tile = (int64_t)(chunk - args.first_chunk[t]) * kWaves + wave;
  if (cancelled) {  // a cancelled step still clears the gradients it was asked to clear
    zero_tile<GT, G::kEpl>(T.g, tile, T.numel, lane);
    return;
  }
  const int64_t begin = tile * G::kTile;
  if (begin >= T.numel) {  // wave past the end of the tensor: only help with the tables
    setup_tables<SR>(lds, tid, slot);
    return;
  }
  const uint32_t salt = !SR ? 0u : EXT ? step_salt(args.sr_salt[t], args.go, args.seed_lo, args.seed_hi) : args.sr_salt[t];
  const StepConsts sc = EXT ? step_consts(args.sc, args.go) : args.sc;
  if (begin + G::kTile <= T.numel)
    process_tile<PT, GT, true, EXT, false, SR, kTileWide, EXACT>(T, begin, lane, wave, tid, sc, lds, slot, gscale, zero_g, salt);
  else
    process_tile<PT, GT, false, EXT, false, SR, kTileWide, EXACT>(T, begin, lane, wave, tid, sc, lds, slot, gscale, zero_g, salt);
}

// ---------------------------------------------------------------------------
// rank-1 scaling of the second moment: the update kernels (statistics, commit and the folds
// for tensors of more dimensions: q4adamw_rank1.h)
// ---------------------------------------------------------------------------
// FORM: how a tile lies in its matrix: kTileWide (rows of at least a tile, multiples of 8),
// kTileNarrow (shorter rows, multiples of 8), kTileAny (rows of any length)
template <int PT, int GT, bool EXT, bool SR, int FORM, bool EXACT>
__global__ __launch_bounds__(kThreads) void fused_4bit_rank1_kernel(const Rank1Args args) {
  using G = Geometry<PT, GT>;
  __shared__ uint2 lds[kLdsEntries];
  const int tid = threadIdx.x;
  const TableSlot slot = request_table_slot<SR>(tid);
  const uint32_t chunk = args.chunk_base + (blockIdx.x & 7u) * args.chunks_per_xcd + (blockIdx.x >> 3);
  if (chunk >= args.nchunks) return;
  float gscale = 1.0f;
  const bool cancelled = EXT && !grad_ops_begin(args.go, gscale);
  const bool zero_g = EXT && args.go.zero != 0u;
  if (cancelled && !zero_g) return;
  const int t = find_tensor(args, chunk);
  const Rank1Desc &T = args.desc[t];
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const int64_t tile = (int64_t)(chunk - args.first_chunk[t]) * kWaves + wave;
  if (cancelled) {
    zero_tile<GT, G::kEpl>(T.g, tile, T.numel, lane);
    return;
  }
  const int64_t begin = tile * G::kTile;
  if (begin >= T.numel) {
    setup_tables<SR>(lds, tid, slot);
    return;
  }
  const uint32_t salt = !SR ? 0u : EXT ? step_salt(args.sr_salt[t], args.go, args.seed_lo, args.seed_hi) : args.sr_salt[t];
  const StepConsts sc = EXT ? step_consts(args.sc, args.go) : args.sc;
  if (begin + G::kTile <= T.numel)
    process_tile<PT, GT, true, EXT, true, SR, FORM, EXACT>(T, begin, lane, wave, tid, sc, lds, slot, gscale, zero_g, salt);
  else
    process_tile<PT, GT, false, EXT, true, SR, FORM, EXACT>(T, begin, lane, wave, tid, sc, lds, slot, gscale, zero_g, salt);
}

// The same for matrices whose rows are a whole number of quantization blocks and at least
// two tiles long: a chunk is one tile's columns of four consecutive rows, one row per wave,
// and tiles start at the beginning of a row, so that the last tile of a row may be a partial
// one (whole blocks; its other lanes are idle).  T.div_magic / div_shift divide by the number
// of tiles in a row.
template <int PT, int GT, bool EXT, bool SR, bool EXACT>
__global__ __launch_bounds__(kThreads) void fused_4bit_rank1_rows_kernel(const Rank1Args args) {
  using G = Geometry<PT, GT>;
  constexpr int N = G::kEpl;
  __shared__ uint2 lds[kLdsEntries];
  __shared__ __attribute__((aligned(16))) float columns[3 * G::kTile];
  const int tid = threadIdx.x;
  const TableSlot slot = request_table_slot<SR>(tid);
  const uint32_t chunk = args.chunk_base + (blockIdx.x & 7u) * args.chunks_per_xcd + (blockIdx.x >> 3);
  if (chunk >= args.nchunks) return;
  float gscale = 1.0f;
  const bool cancelled = EXT && !grad_ops_begin(args.go, gscale);
  const bool zero_g = EXT && args.go.zero != 0u;
  if (cancelled && !zero_g) return;
  const int t = find_tensor(args, chunk);
  const Rank1Desc &T = args.desc[t];
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
  const uint32_t local = chunk - args.first_chunk[t];
  const uint32_t cols = (uint32_t)T.cols;
  const uint32_t tiles_per_row = (cols + (uint32_t)G::kTile - 1u) / (uint32_t)G::kTile;
  const uint32_t row_group = fast_div(local, T.div_magic, T.div_shift);
  const uint32_t col_tile = local - row_group * tiles_per_row;
  RowsTile rt;
  rt.row = (int64_t)row_group * kWaves + wave;
  rt.col0 = col_tile * (uint32_t)G::kTile;
  rt.width = cols - rt.col0 < (uint32_t)G::kTile ? cols - rt.col0 : (uint32_t)G::kTile;
  rt.columns = columns;
  const bool idle = rt.row >= T.rows;   // the last rows of a matrix whose row count is no multiple of four
  const int64_t begin = rt.row * T.cols + rt.col0;   // the tile's first element
  const bool whole = rt.width == (uint32_t)G::kTile;
  if (cancelled) {
    if (!idle && (uint32_t)lane * N < rt.width)
      zero_elems<GT, N, true>(static_cast<char *>(const_cast<void *>(T.g)) + begin * (GT ? 2 : 4), (uint32_t)lane * N, N);
    return;
  }
  // this thread's share of the columns' maxima: N / 4 consecutive columns (zeros past the row's end)
  const uint32_t share = rt.col0 + (uint32_t)tid * (N / 4);
  rt.share_old = rt.share_new = make_float2(0.0f, 0.0f);
  if (whole || share < cols) {
    if (N == 4) {
      rt.share_old.x = as_global<const float>(T.cmax)[share];
      rt.share_new.x = as_global<const float>(T.cmax_next)[share];
    } else {
      rt.share_old = make_float2(as_global<const float>(T.cmax)[share], as_global<const float>(T.cmax)[share + 1]);
      rt.share_new = make_float2(as_global<const float>(T.cmax_next)[share], as_global<const float>(T.cmax_next)[share + 1]);
    }
  }
  if (idle) {  // only help with the tables and the columns
    stage_columns<N>(rt, tid);
    setup_tables<SR>(lds, tid, slot);
    return;
  }
  const uint32_t salt = !SR ? 0u : EXT ? step_salt(args.sr_salt[t], args.go, args.seed_lo, args.seed_hi) : args.sr_salt[t];
  const StepConsts sc = EXT ? step_consts(args.sc, args.go) : args.sc;
  if (__builtin_expect(whole, 1))
    process_tile<PT, GT, true, EXT, true, SR, kTileRows, EXACT>(T, begin, lane, wave, tid, sc, lds, slot, gscale, zero_g, salt, &rt);
  else
    process_tile<PT, GT, true, EXT, true, SR, kTileRowsLast, EXACT>(T, begin, lane, wave, tid, sc, lds, slot, gscale, zero_g, salt, &rt);
}

}  // namespace q4
