// Memory-system probes for bench.py: what this GPU's HBM delivers to kernels that move bytes
// the way the fused step moves them, with none of its arithmetic.  They answer "how far is the
// step kernel from what its own access pattern can reach", which the published peak cannot.
//
//   copy          every lane loads 16 bytes and stores 16 bytes (1:1 read:write)
//   read          every lane loads 16 bytes, nothing is written
//   step streams  the fused step's seven streams in its own geometry: per lane one access of
//                 p and of g (16 bytes of the wider one), 2 or 4 bytes of each moment's codes,
//                 per 128 elements one fp32 scale of each moment; p, the codes and the scales
//                 are written back.  fp32 p / bf16 g: 7.0625 bytes read and 5.0625 written per
//                 element, the step's own ratio.  The code and scale streams can be left out,
//                 which shows what these small streams cost the large ones.
//
// All three use the step's launch shape (one tile per wave64, four waves per workgroup,
// workgroups dealt to the XCDs so that each walks a contiguous eighth), its buffer
// instructions and its cache policy (q4adamw_device.h), so a difference between the step and
// its probe is the step's arithmetic and tables, not its addressing.
//
// Build: hipcc --offload-arch=gfx950 -O3 -shared -fPIC (quantfour_adamw_cuda_amd/build.py).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/q4probe.h"
#include "q4adamw_device.h"

namespace q4 {

struct ProbeArgs {
  void *a;            // copy: destination; read: sink; step streams: p
  const void *b;      // copy / read: source; step streams: g
  uint8_t *m, *v;     // step streams: packed codes
  float *sm, *sv;     // step streams: block scales
  uint64_t units;     // copy / read: 16-byte units; step streams: elements
  uint32_t nchunks;
  uint32_t chunks_per_xcd;
};

__device__ __forceinline__ uint32_t probe_chunk(const ProbeArgs &a) {
  return (blockIdx.x & 7u) * a.chunks_per_xcd + (blockIdx.x >> 3);
}

// mode 0: copy, mode 1: read only (the sink is written by no lane in practice: the test
// below cannot be decided at compile time and holds for no data the bench feeds)
template <int MODE>
__global__ __launch_bounds__(kThreads) void probe_move_kernel(const ProbeArgs a) {
  const uint32_t chunk = probe_chunk(a);
  if (chunk >= a.nchunks) return;
  const uint64_t unit0 = (uint64_t)chunk * kThreads;   // first 16-byte unit of the workgroup
  const uint32_t tid = threadIdx.x;
  if (unit0 + tid >= a.units) return;
  const char *src = static_cast<const char *>(a.b) + unit0 * 16;
  const u32x4 w = __builtin_amdgcn_raw_buffer_load_b128(tile_rsrc(src), tid * 16u, 0, MODE ? kNtReadOnly : kNt);
  if (MODE == 0) {
    char *dst = static_cast<char *>(a.a) + unit0 * 16;
    __builtin_amdgcn_raw_buffer_store_b128(w, tile_rsrc(dst), tid * 16u, 0, kNt);
  } else if ((w.x ^ w.y ^ w.z ^ w.w) == 0x9E3779B9u && w.x == 0x7F4A7C15u) {
    as_global<uint32_t>(a.a)[0] = w.x;
  }
}

// PB, GB: bytes per element of p and g (4 or 2).  Full tiles only (the host rounds down).
// CODES, SCALES: with the moments' code streams / scale streams (without them the probe shows
// what those small streams cost the large ones).
template <int PB, int GB, bool CODES, bool SCALES>
__global__ __launch_bounds__(kThreads) void probe_step_streams_kernel(const ProbeArgs a) {
  constexpr int N = (PB == 2 && GB == 2) ? 8 : 4;          // elements per lane, as Geometry<PT, GT>
  constexpr int kTile = 64 * N;
  constexpr int kLanesPerBlock = Q4ADAMW_BLOCK / N;
  constexpr int kBlocksPerTile = kTile / Q4ADAMW_BLOCK;
  const uint32_t chunk = probe_chunk(a);
  if (chunk >= a.nchunks) return;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int64_t tile = (int64_t)chunk * kWaves + wave;
  const int64_t tb = tile * kTile;
  if (tb + kTile > (int64_t)a.units) return;
  char *p_tile = static_cast<char *>(a.a) + tb * PB;
  const char *g_tile = static_cast<const char *>(a.b) + tb * GB;
  uint8_t *m_tile = a.m + (tb >> 1), *v_tile = a.v + (tb >> 1);
  float *sm_tile = a.sm + tile * kBlocksPerTile, *sv_tile = a.sv + tile * kBlocksPerTile;
  const uint32_t e0 = (uint32_t)lane * N, blk = (uint32_t)lane / kLanesPerBlock, code_off = (uint32_t)lane * (N / 2);

  // loads, in the step's order: p, g, codes, scales
  u32x4 pw = {0u, 0u, 0u, 0u}, gw = {0u, 0u, 0u, 0u};
  if (N * PB == 16) {
    pw = __builtin_amdgcn_raw_buffer_load_b128(tile_rsrc(p_tile), e0 * PB, 0, kNt);
  } else {
    const u32x2 t = __builtin_amdgcn_raw_buffer_load_b64(tile_rsrc(p_tile), e0 * PB, 0, kNt);
    pw.x = t.x; pw.y = t.y;
  }
  if (N * GB == 16) {
    gw = __builtin_amdgcn_raw_buffer_load_b128(tile_rsrc(g_tile), e0 * GB, 0, kNt);
  } else {
    const u32x2 t = __builtin_amdgcn_raw_buffer_load_b64(tile_rsrc(g_tile), e0 * GB, 0, kNt);
    gw.x = t.x; gw.y = t.y;
  }
  uint32_t mw = 0u, vw = 0u, s_m = 0u, s_v = 0u;
  if (CODES) {
    if (N == 4) {
      mw = __builtin_amdgcn_raw_buffer_load_b16(tile_rsrc(m_tile), code_off, 0, kNt);
      vw = __builtin_amdgcn_raw_buffer_load_b16(tile_rsrc(v_tile), code_off, 0, kNt);
    } else {
      mw = __builtin_amdgcn_raw_buffer_load_b32(tile_rsrc(m_tile), code_off, 0, kNt);
      vw = __builtin_amdgcn_raw_buffer_load_b32(tile_rsrc(v_tile), code_off, 0, kNt);
    }
  }
  if (SCALES) {
    s_m = __builtin_amdgcn_raw_buffer_load_b32(tile_rsrc(sm_tile), blk * 4u, 0, 0);
    s_v = __builtin_amdgcn_raw_buffer_load_b32(tile_rsrc(sv_tile), blk * 4u, 0, 0);
  }

  // every stored value depends on every loaded one, at the price of a few integer operations
  const uint32_t mix = gw.x ^ gw.y ^ gw.z ^ gw.w ^ mw ^ vw ^ s_m ^ s_v;
  pw.x ^= mix; pw.y += mix; pw.z ^= mix; pw.w += mix;
  if (N * PB == 16) {
    __builtin_amdgcn_raw_buffer_store_b128(pw, tile_rsrc(p_tile), e0 * PB, 0, kNt);
  } else {
    const u32x2 t = {pw.x, pw.y};
    __builtin_amdgcn_raw_buffer_store_b64(t, tile_rsrc(p_tile), e0 * PB, 0, kNt);
  }
  if (CODES) {
    if (N == 4) {
      __builtin_amdgcn_raw_buffer_store_b16((uint16_t)(mw ^ pw.x), tile_rsrc(m_tile), code_off, 0, kNt);
      __builtin_amdgcn_raw_buffer_store_b16((uint16_t)(vw ^ pw.y), tile_rsrc(v_tile), code_off, 0, kNt);
    } else {
      __builtin_amdgcn_raw_buffer_store_b32(mw ^ pw.x, tile_rsrc(m_tile), code_off, 0, kNt);
      __builtin_amdgcn_raw_buffer_store_b32(vw ^ pw.y, tile_rsrc(v_tile), code_off, 0, kNt);
    }
  }
  if (SCALES && (lane & (kLanesPerBlock - 1)) == 0) {
    __builtin_amdgcn_raw_buffer_store_b32(s_m ^ pw.x, tile_rsrc(sm_tile), blk * 4u, 0, 0);
    __builtin_amdgcn_raw_buffer_store_b32(s_v ^ pw.y, tile_rsrc(sv_tile), blk * 4u, 0, 0);
  }
}

static int probe_launch(ProbeArgs &a, uint64_t chunks, void (*kernel)(const ProbeArgs), void *stream) {
  if (chunks == 0) return 0;
  if (chunks > 0x7ffffff0ull) return Q4PROBE_ERR_ARG;
  a.nchunks = (uint32_t)chunks;
  a.chunks_per_xcd = (uint32_t)((chunks + 7) / 8);
  hipLaunchKernelGGL(kernel, dim3(a.chunks_per_xcd * 8u), dim3(kThreads), 0, static_cast<hipStream_t>(stream), a);
  return (int)hipGetLastError();
}

typedef void (*ProbeKernel)(const ProbeArgs);

template <bool CODES, bool SCALES>
static ProbeKernel pick_streams(bool p16, bool g16) {
  if (p16) return g16 ? probe_step_streams_kernel<2, 2, CODES, SCALES> : probe_step_streams_kernel<2, 4, CODES, SCALES>;
  return g16 ? probe_step_streams_kernel<4, 2, CODES, SCALES> : probe_step_streams_kernel<4, 4, CODES, SCALES>;
}

}  // namespace q4

using namespace q4;

extern "C" {

int q4probe_copy(void *dst, const void *src, uint64_t bytes, void *stream) {
  if (!dst || !src || (reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src) | bytes) & 15u)
    return Q4PROBE_ERR_ARG;
  ProbeArgs a = {};
  a.a = dst;
  a.b = src;
  a.units = bytes / 16;
  return probe_launch(a, (a.units + kThreads - 1) / kThreads, probe_move_kernel<0>, stream);
}

int q4probe_read(const void *src, uint64_t bytes, void *sink4, void *stream) {
  if (!src || !sink4 || (reinterpret_cast<uintptr_t>(src) | bytes) & 15u || reinterpret_cast<uintptr_t>(sink4) & 3u)
    return Q4PROBE_ERR_ARG;
  ProbeArgs a = {};
  a.a = sink4;
  a.b = src;
  a.units = bytes / 16;
  return probe_launch(a, (a.units + kThreads - 1) / kThreads, probe_move_kernel<1>, stream);
}

int q4probe_step_streams(void *p, const void *g, uint8_t *exp_avg, uint8_t *exp_avg_sq, float *exp_avg_scale,
                         float *exp_avg_sq_scale, uint64_t numel, int p_dtype, int g_dtype, int streams,
                         void *stream) {
  if (!p || !g || !exp_avg || !exp_avg_sq || !exp_avg_scale || !exp_avg_sq_scale) return Q4PROBE_ERR_ARG;
  if (p_dtype < 0 || p_dtype > 2 || g_dtype < 0 || g_dtype > 2) return Q4PROBE_ERR_ARG;
  if ((reinterpret_cast<uintptr_t>(p) | reinterpret_cast<uintptr_t>(g)) & 15u) return Q4PROBE_ERR_ARG;
  if ((reinterpret_cast<uintptr_t>(exp_avg) | reinterpret_cast<uintptr_t>(exp_avg_sq) |
       reinterpret_cast<uintptr_t>(exp_avg_scale) | reinterpret_cast<uintptr_t>(exp_avg_sq_scale)) & 3u)
    return Q4PROBE_ERR_ARG;
  const bool p16 = p_dtype != 0, g16 = g_dtype != 0;
  const uint64_t chunk_elems = (p16 && g16 ? 512u : 256u) * kWaves;
  ProbeArgs a = {};
  a.a = p;
  a.b = g;
  a.m = exp_avg;
  a.v = exp_avg_sq;
  a.sm = exp_avg_scale;
  a.sv = exp_avg_sq_scale;
  a.units = numel;
  if (streams < 0 || streams > 3) return Q4PROBE_ERR_ARG;
  const bool codes = streams & Q4PROBE_CODES, scales = streams & Q4PROBE_SCALES;
  const ProbeKernel kernel = codes ? (scales ? pick_streams<true, true>(p16, g16) : pick_streams<true, false>(p16, g16))
                                          : (scales ? pick_streams<false, true>(p16, g16) : pick_streams<false, false>(p16, g16));
  return probe_launch(a, numel / chunk_elems, kernel, stream);   // whole chunks only
}

}  // extern "C"
