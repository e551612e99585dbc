/*
 * q4probe -- memory-system probes that bench.py times beside the fused 4-bit AdamW step
 * (libq4probe.so, built from quantfour_adamw_cuda_amd/csrc/q4stream_probe.hip).  No
 * counterpart in the reference: they exist so that the bench can report what this GPU's HBM
 * delivers to kernels that move the step's bytes in the step's access pattern with none of
 * its arithmetic -- the ceiling the step kernel is measured against besides the published
 * peak.  Not part of the optimizer: nothing in the step path loads this library.
 *
 * All pointers are device pointers, 16-byte aligned unless said otherwise; work is enqueued
 * on `stream` (a hipStream_t, NULL = default stream); return 0, Q4PROBE_ERR_ARG or a
 * hipError_t.  The buffers' contents are overwritten with meaningless values.
 */
#ifndef Q4PROBE_H
#define Q4PROBE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define Q4PROBE_ERR_ARG (-1)

/* dst[i] = src[i]: every lane loads 16 bytes and stores 16 bytes.  bytes % 16 == 0. */
int q4probe_copy(void *dst, const void *src, uint64_t bytes, void *stream);

/* Reads src and writes nothing (sink4: four device bytes that stay as they are). */
int q4probe_read(const void *src, uint64_t bytes, void *sink4, void *stream);

/*
 * The seven streams of the fused step (q4adamw_fused_4bit) in its geometry and with its
 * cache policy, without its arithmetic: reads p, g, both moments' packed codes and block
 * scales, writes p, the codes and the scales.  Arguments as q4adamw_fused_4bit; only whole
 * workgroups' worth of elements (1024, or 2048 when p and g are both 16-bit types) are
 * touched, so pass a multiple of 2048.  streams: Q4PROBE_CODES | Q4PROBE_SCALES for all seven;
 * without a bit the two moments' streams of that kind are neither read nor written.
 */
#define Q4PROBE_CODES 1
#define Q4PROBE_SCALES 2
int q4probe_step_streams(void *p, const void *g, uint8_t *exp_avg, uint8_t *exp_avg_sq,
                         float *exp_avg_scale, float *exp_avg_sq_scale, uint64_t numel, int p_dtype,
                         int g_dtype, int streams, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* Q4PROBE_H */
