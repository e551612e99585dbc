/*
 * Host code of the C ABI under AddressSanitizer and UndefinedBehaviorSanitizer, without a
 * GPU: the program links a build of csrc/q4adamw.hip whose host code is sanitized and walks
 *   - the host-only entry points (tables, derived scalars, bucket-table probes, noise salts)
 *   - every refusal an entry point makes before it launches anything (null pointers,
 *     misalignment, negative and oversized shapes, hyper-parameters out of range, workspaces
 *     too small), and the calls that have nothing to do (empty lists, zero elements)
 * and the scalar C oracle (oracle/q4_oracle.c, compiled with the same sanitizers) on sizes
 * with tails and all-zero blocks.  No kernel is launched.  tests/test_sanitizers.py builds
 * and runs it; the sanitizers abort on a finding, the program prints "host_sanitize: ok".
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "q4adamw.h"

void q4o_step_quant(void *p, const void *g, uint8_t *m_codes, uint8_t *v_codes, float *m_scale,
                    float *v_scale, int64_t numel, int p_dtype, int g_dtype, float beta1,
                    float beta2, float lr, float weight_decay, float eps, float step);
void q4o_step_unquant(void *p, const void *g, float *m, float *v, int64_t numel, int p_dtype,
                      int g_dtype, float beta1, float beta2, float lr, float weight_decay,
                      float eps, float step);
void q4o_quant(const float *x, int64_t numel, int which, uint8_t *codes, float *scale);
void q4o_dequant(const uint8_t *codes, const float *scale, int64_t numel, int which, float *out);
void q4o_derive_scalars(float beta1, float beta2, float lr, float weight_decay, float step, float *out6);

#define TRUE_(cond)                                                        \
  do {                                                                     \
    if (!(cond)) {                                                         \
      fprintf(stderr, "%s:%d %s does not hold\n", __FILE__, __LINE__, #cond); \
      exit(1);                                                             \
    }                                                                      \
  } while (0)

#define EXPECT(call, want)                                                                     \
  do {                                                                                         \
    int rc_ = (call);                                                                          \
    if (rc_ != (want)) {                                                                       \
      fprintf(stderr, "%s:%d %s returned %d (%s), expected %d\n", __FILE__, __LINE__, #call, rc_, \
              q4adamw_last_error(), (want));                                                   \
      exit(1);                                                                                 \
    }                                                                                          \
    if ((want) != 0 && strlen(q4adamw_last_error()) == 0) {                                    \
      fprintf(stderr, "%s:%d no error message\n", __FILE__, __LINE__);                         \
      exit(1);                                                                                 \
    }                                                                                          \
  } while (0)

static const float B1 = 0.9f, B2 = 0.999f, LR = 1e-3f, WD = 0.01f, EPS = 1e-8f;

static void host_only_entry_points(void) {
  float qmap[16], qmid[15], a[6], b[6];
  for (int which = 0; which < 2; ++which) q4adamw_tables(which, qmap, qmid);
  for (int step = 1; step < 2000; step += 37) {
    q4adamw_derive_scalars(B1, B2, LR, WD, (float)step, a);
    q4o_derive_scalars(B1, B2, LR, WD, (float)step, b);
    if (memcmp(a, b, sizeof a) != 0) {
      fprintf(stderr, "derived scalars differ at step %d\n", step);
      exit(1);
    }
  }
  uint32_t pair[2];
  for (uint32_t i = 0; i < 2048; ++i) EXPECT(q4adamw_mtable_entry(i, pair), 0);
  EXPECT(q4adamw_mtable_entry(2048, pair), Q4ADAMW_ERR_ARG);
  EXPECT(q4adamw_mtable_entry(0, NULL), Q4ADAMW_ERR_ARG);
  for (uint32_t i = 0; i < 256; ++i) {
    const int bkt = q4adamw_mtable_half_bucket(i);
    if (bkt < 0 || bkt >= 2048) {
      fprintf(stderr, "half bucket %u -> %d\n", i, bkt);
      exit(1);
    }
  }
  EXPECT(q4adamw_mtable_half_bucket(256), Q4ADAMW_ERR_ARG);
  for (uint32_t i = 0; i < 256; ++i) EXPECT(q4adamw_sr_bucket_entry(i, pair), 0);
  EXPECT(q4adamw_sr_bucket_entry(256, pair), Q4ADAMW_ERR_ARG);
  EXPECT(q4adamw_sr_bucket_entry(0, NULL), Q4ADAMW_ERR_ARG);
  {
    float affine[2];
    for (uint32_t k = 0; k <= 16; ++k) EXPECT(q4adamw_sr_affine_entry(k, affine), 0);
    EXPECT(q4adamw_sr_affine_entry(17, affine), Q4ADAMW_ERR_ARG);
    EXPECT(q4adamw_sr_affine_entry(0, NULL), Q4ADAMW_ERR_ARG);
  }
  uint32_t acc = 0;
  for (uint32_t s = 0; s < 1000; ++s) acc ^= q4adamw_sr_tensor_salt(0xFFFFFFFFFFFFFFFFull - s, (float)(s + 1), s * 2654435761u);
  if (acc == 0) printf("(salts xor to zero)\n");
  if (q4adamw_version() < 1000 || q4adamw_release() != 0) exit(1);
}

static void refusals(void) {
  /* host memory stands in for device memory: every call below returns before a launch */
  float *buf = aligned_alloc(256, 1 << 16);
  uint8_t *codes = (uint8_t *)buf + 32768;
  float *scales = buf + 12000;
  const int F = Q4ADAMW_FP32, H = Q4ADAMW_BF16;
  EXPECT(q4adamw_fused_4bit(buf, buf + 2048, codes, codes + 2048, scales, scales + 64, 0, F, F, B1, B2, LR, WD, EPS, 1.0f, NULL), 0);
  EXPECT(q4adamw_fused_4bit((float *)((char *)buf + 2), buf + 2048, codes, codes + 2048, scales, scales + 64, 1000, F, F, B1, B2, LR, WD, EPS, 1.0f, NULL), Q4ADAMW_ERR_ALIGN);
  EXPECT(q4adamw_fused_4bit(buf, buf + 2048, codes + 1, codes + 2048, scales, scales + 64, 1000, F, F, B1, B2, LR, WD, EPS, 1.0f, NULL), Q4ADAMW_ERR_ALIGN);
  EXPECT(q4adamw_fused_4bit(buf, buf + 2048, codes + 2, codes + 2048, scales, scales + 64, 1000, H, H, B1, B2, LR, WD, EPS, 1.0f, NULL), Q4ADAMW_ERR_ALIGN);
  EXPECT(q4adamw_fused_4bit(buf, NULL, codes, codes + 2048, scales, scales + 64, 1000, F, F, B1, B2, LR, WD, EPS, 1.0f, NULL), Q4ADAMW_ERR_ARG);
  EXPECT(q4adamw_fused_4bit(buf, buf + 2048, codes, codes + 2048, scales, scales + 64, -1, F, F, B1, B2, LR, WD, EPS, 1.0f, NULL), Q4ADAMW_ERR_ARG);
  EXPECT(q4adamw_fused_4bit(buf, buf + 2048, codes, codes + 2048, scales, scales + 64, 1000, 3, F, B1, B2, LR, WD, EPS, 1.0f, NULL), Q4ADAMW_ERR_ARG);
  EXPECT(q4adamw_fused_4bit(buf, buf + 2048, codes, codes + 2048, scales, scales + 64, INT64_MAX, F, F, B1, B2, LR, WD, EPS, 1.0f, NULL), Q4ADAMW_ERR_TOO_LARGE);
  const float bad_hyper[][6] = {{1.0f, B2, LR, WD, EPS, 1.0f}, {B1, 0.0f, LR, WD, EPS, 1.0f}, {B1, B2, 0.0f, WD, EPS, 1.0f},
                                {B1, B2, LR, -1.0f, EPS, 1.0f}, {B1, B2, LR, WD, 0.0f, 1.0f}, {B1, B2, LR, WD, EPS, 0.5f},
                                {NAN, B2, LR, WD, EPS, 1.0f}, {B1, B2, NAN, WD, EPS, 1.0f}, {B1, B2, LR, WD, EPS, NAN}};
  for (size_t k = 0; k < sizeof bad_hyper / sizeof bad_hyper[0]; ++k) {
    const float *h = bad_hyper[k];
    EXPECT(q4adamw_fused_4bit(buf, buf + 2048, codes, codes + 2048, scales, scales + 64, 1000, F, F, h[0], h[1], h[2], h[3], h[4], h[5], NULL), Q4ADAMW_ERR_HYPER);
    EXPECT(q4adamw_fused_single_tensor(buf, buf + 2048, buf + 4096, buf + 6144, 1000, F, F, h[0], h[1], h[2], h[3], h[4], h[5], NULL), Q4ADAMW_ERR_HYPER);
  }
  /* grids: a batch beyond what one grid holds (2^32 work-items: 2^24 - 8 workgroups of 256
     threads once rounded to a multiple of 8) is dealt to several */
  {
    uint64_t bases[8], counts[8];
    const uint64_t limit = (1ull << 24) - 8;
    TRUE_(q4adamw_grid_plan(0, 256, bases, counts, 8) == 0);
    TRUE_(q4adamw_grid_plan(limit - 1, 256, bases, counts, 8) == 1);
    TRUE_(q4adamw_grid_plan(limit, 256, bases, counts, 8) == 1);
    TRUE_(bases[0] == 0 && counts[0] == limit);
    TRUE_(q4adamw_grid_plan(limit + 1, 256, bases, counts, 8) == 2);
    TRUE_(bases[1] == limit && counts[1] == 1);
    TRUE_(q4adamw_grid_plan((1ull << 24) - 1, 256, bases, counts, 8) == 2);      /* what HIP itself would still take */
    TRUE_(q4adamw_grid_plan(1ull << 24, 256, bases, counts, 8) == 2);
    TRUE_(q4adamw_grid_plan((1ull << 24) + 1, 256, bases, counts, 8) == 2);
    TRUE_(bases[1] + counts[1] == (1ull << 24) + 1);
    TRUE_(q4adamw_grid_plan(0x7ffffff0ull, 256, bases, counts, 2) == 129);        /* more grids than the arrays hold */
    EXPECT(q4adamw_grid_plan(0x7ffffff1ull, 256, bases, counts, 8), Q4ADAMW_ERR_TOO_LARGE);
    EXPECT(q4adamw_grid_plan(10, 32, bases, counts, 8), Q4ADAMW_ERR_ARG);
    EXPECT(q4adamw_grid_plan(10, 256, NULL, counts, 8), Q4ADAMW_ERR_ARG);
    q4adamw_set_grid_limit(70);                 /* rounded down to 64 */
    TRUE_(q4adamw_grid_plan(200, 256, bases, counts, 8) == 4);
    TRUE_(bases[3] == 192 && counts[3] == 8 && counts[0] == 64);
    q4adamw_set_grid_limit(3);                  /* below 8: ignored */
    TRUE_(q4adamw_grid_plan(200, 256, bases, counts, 8) == 1);
    q4adamw_set_grid_limit(0);
    TRUE_(q4adamw_grid_plan(200, 256, bases, counts, 8) == 1);
    /* a tensor beyond one grid is taken (the launch itself fails here: no device), one beyond a batch's 31-bit chunk index is not */
    EXPECT(q4adamw_fused_4bit(buf, buf + 2048, codes, codes + 2048, scales, scales + 64, (int64_t)0x7ffffff0ll * 1024 + 1, F, F, B1, B2, LR, WD, EPS, 1.0f, NULL), Q4ADAMW_ERR_TOO_LARGE);
  }
  /* lists */
  q4adamw_tensor t[2];
  memset(t, 0, sizeof t);
  EXPECT(q4adamw_fused_4bit_multi(t, 2, F, F, B1, B2, LR, WD, EPS, 1.0f, NULL), 0);      /* two empty tensors */
  EXPECT(q4adamw_fused_4bit_multi(NULL, 0, F, F, B1, B2, LR, WD, EPS, 1.0f, NULL), 0);
  EXPECT(q4adamw_fused_4bit_multi(NULL, 2, F, F, B1, B2, LR, WD, EPS, 1.0f, NULL), Q4ADAMW_ERR_ARG);
  EXPECT(q4adamw_fused_4bit_multi(t, -1, F, F, B1, B2, LR, WD, EPS, 1.0f, NULL), Q4ADAMW_ERR_ARG);
  t[1].numel = 10;   /* pointers still null */
  EXPECT(q4adamw_fused_4bit_multi(t, 2, F, F, B1, B2, LR, WD, EPS, 1.0f, NULL), Q4ADAMW_ERR_ARG);
  EXPECT(q4adamw_fused_4bit_multi_sr(t, 2, NULL, 7, F, F, B1, B2, LR, WD, EPS, 1.0f, NULL, NULL), Q4ADAMW_ERR_ARG);
  q4adamw_grad_options opt = {1.0f, 0, (const float *)((const char *)buf + 2), NULL};
  t[1].numel = 0;
  EXPECT(q4adamw_fused_4bit_multi_ex(t, 2, F, F, B1, B2, LR, WD, EPS, 1.0f, &opt, NULL), Q4ADAMW_ERR_ALIGN);
  opt.grad_scale_dev = NULL;
  opt.skip_if_nonzero = (const float *)((const char *)buf + 1);
  EXPECT(q4adamw_fused_4bit_multi_ex(t, 2, F, F, B1, B2, LR, WD, EPS, 1.0f, &opt, NULL), Q4ADAMW_ERR_ALIGN);
  q4adamw_small_tensor st[1];
  memset(st, 0, sizeof st);
  EXPECT(q4adamw_fused_single_tensor_multi(st, 1, F, F, B1, B2, LR, WD, EPS, 1.0f, NULL), 0);
  st[0].numel = 5;
  EXPECT(q4adamw_fused_single_tensor_multi(st, 1, F, F, B1, B2, LR, WD, EPS, 1.0f, NULL), Q4ADAMW_ERR_ARG);
  st[0].p = (char *)buf + 2; st[0].g = buf; st[0].exp_avg = buf; st[0].exp_avg_sq = buf;
  EXPECT(q4adamw_fused_single_tensor_multi(st, 1, F, F, B1, B2, LR, WD, EPS, 1.0f, NULL), Q4ADAMW_ERR_ALIGN);
  /* rank-1 */
  q4adamw_rank1_tensor r[1];
  memset(r, 0, sizeof r);
  EXPECT(q4adamw_fused_4bit_rank1_multi(r, 1, F, F, B1, B2, LR, WD, EPS, 1.0f, NULL, NULL), 0);   /* 0 x 0 */
  r[0].rows = 4; r[0].cols = 520;
  EXPECT(q4adamw_fused_4bit_rank1_multi(r, 1, F, F, B1, B2, LR, WD, EPS, 1.0f, NULL, NULL), Q4ADAMW_ERR_ARG);   /* null pointers */
  r[0].cols = 1;
  EXPECT(q4adamw_fused_4bit_rank1_multi(r, 1, F, F, B1, B2, LR, WD, EPS, 1.0f, NULL, NULL), Q4ADAMW_ERR_ARG);   /* one column */
  r[0].rows = (int64_t)1 << 20; r[0].cols = 4100;   /* rows of any length: fewer than 2^32 elements */
  EXPECT(q4adamw_fused_4bit_rank1_multi_sr(r, 1, NULL, 1, F, F, B1, B2, LR, WD, EPS, 1.0f, NULL, NULL), Q4ADAMW_ERR_TOO_LARGE);
  TRUE_(q4adamw_rank1_form(100, 516, 0) == 3 && q4adamw_rank1_form(100, 8, 1) == 3 && q4adamw_rank1_form(4096, 4096, 0) == 0);
  EXPECT(q4adamw_rank1_form(0, 16, 0), Q4ADAMW_ERR_ARG);
  r[0].rows = -1;
  EXPECT(q4adamw_fused_4bit_rank1_multi(r, 1, F, F, B1, B2, LR, WD, EPS, 1.0f, NULL, NULL), Q4ADAMW_ERR_ARG);
  r[0].rows = (int64_t)1 << 40; r[0].cols = 1024;
  EXPECT(q4adamw_fused_4bit_rank1_multi(r, 1, F, F, B1, B2, LR, WD, EPS, 1.0f, NULL, NULL), Q4ADAMW_ERR_TOO_LARGE);
  /* leading dimensions: their product must be rows, their statistics must be there */
  r[0].rows = 6; r[0].cols = 16;
  r[0].p = buf; r[0].g = buf + 1024; r[0].exp_avg = codes; r[0].exp_avg_sq = codes + 1024; r[0].exp_avg_scale = scales;
  r[0].row_max = scales + 64; r[0].row_max_next = scales + 128; r[0].col_max = buf + 2048; r[0].col_max_next = buf + 3072;
  r[0].lead_dims = 4;
  EXPECT(q4adamw_fused_4bit_rank1_multi(r, 1, F, F, B1, B2, LR, WD, EPS, 1.0f, NULL, NULL), Q4ADAMW_ERR_ARG);
  r[0].lead_dims = 2; r[0].lead_shape[0] = 2; r[0].lead_shape[1] = 3;
  EXPECT(q4adamw_fused_4bit_rank1_multi(r, 1, F, F, B1, B2, LR, WD, EPS, 1.0f, NULL, NULL), Q4ADAMW_ERR_ARG);   /* no statistics */
  r[0].lead_max[0] = scales + 192; r[0].lead_max[1] = scales + 200; r[0].lead_max_next[0] = scales + 208;
  r[0].lead_max_next[1] = (float *)((char *)(scales + 216) + 2);
  EXPECT(q4adamw_fused_4bit_rank1_multi(r, 1, F, F, B1, B2, LR, WD, EPS, 1.0f, NULL, NULL), Q4ADAMW_ERR_ALIGN);
  r[0].lead_max_next[1] = scales + 216; r[0].lead_shape[1] = 4;
  EXPECT(q4adamw_fused_4bit_rank1_multi(r, 1, F, F, B1, B2, LR, WD, EPS, 1.0f, NULL, NULL), Q4ADAMW_ERR_ARG);   /* 2 x 4 != 6 */
  EXPECT(q4adamw_quantize_rank1_scaled(buf, 4, -12, scales, scales + 64, codes, NULL), Q4ADAMW_ERR_ARG);
  EXPECT(q4adamw_quantize_rank1_scaled(buf, 4, 16, NULL, scales + 64, codes, NULL), Q4ADAMW_ERR_ARG);
  EXPECT(q4adamw_quantize_rank1_scaled(buf, 0, 16, scales, scales + 64, codes, NULL), 0);
  EXPECT(q4adamw_bias_table(0.9f, 0.999f, 1, 4, buf), 0);
  EXPECT(q4adamw_bias_table(0.9f, 0.999f, 0, 4, buf), Q4ADAMW_ERR_ARG);
  EXPECT(q4adamw_device_step(NULL, buf, 1, 4, NULL, B1, B2, LR, WD, EPS, NULL, buf + 64, NULL), Q4ADAMW_ERR_ARG);
  EXPECT(q4adamw_device_step(buf, buf + 16, 1, 4, NULL, B1, B2, LR, WD, EPS, NULL, (char *)(buf + 64) + 4, NULL), Q4ADAMW_ERR_ALIGN);
  EXPECT(q4adamw_device_step(buf, buf + 16, 1, 0, NULL, B1, B2, LR, WD, EPS, NULL, buf + 64, NULL), Q4ADAMW_ERR_ARG);
  EXPECT(q4adamw_quantize_rank1(buf, -4, 12, codes, scales, scales + 64, NULL), Q4ADAMW_ERR_ARG);
  EXPECT(q4adamw_quantize_rank1(buf, 0, 16, codes, scales, scales + 64, NULL), 0);
  EXPECT(q4adamw_quantize_rank1(buf, (int64_t)1 << 23, 8, codes, scales, scales + 64, NULL), Q4ADAMW_ERR_TOO_LARGE);
  EXPECT(q4adamw_dequantize_rank1(codes, scales, scales + 64, -2, 16, buf, NULL), Q4ADAMW_ERR_ARG);
  EXPECT(q4adamw_dequantize_rank1(NULL, scales, scales + 64, 2, 16, buf, NULL), Q4ADAMW_ERR_ARG);
  /* gradient norm */
  q4adamw_grad gr[1] = {{buf, 100}};
  EXPECT(q4adamw_grad_norm(gr, 1, F, 1.0f, NULL, 1.0f, NULL, Q4ADAMW_NORM_WORKSPACE_BYTES, buf, NULL), Q4ADAMW_ERR_ARG);
  EXPECT(q4adamw_grad_norm(gr, 1, F, 1.0f, NULL, 1.0f, buf + 1024, 100, buf, NULL), Q4ADAMW_ERR_ARG);
  EXPECT(q4adamw_grad_norm(gr, 1, F, 1.0f, NULL, 1.0f, (char *)(buf + 1024) + 4, Q4ADAMW_NORM_WORKSPACE_BYTES, buf, NULL), Q4ADAMW_ERR_ALIGN);
  gr[0].g = (char *)buf + 2;
  EXPECT(q4adamw_grad_norm(gr, 1, F, 1.0f, NULL, 1.0f, buf + 1024, Q4ADAMW_NORM_WORKSPACE_BYTES, buf, NULL), Q4ADAMW_ERR_ALIGN);
  gr[0].g = NULL;
  EXPECT(q4adamw_grad_norm(gr, 1, H, 1.0f, NULL, 1.0f, buf + 1024, Q4ADAMW_NORM_WORKSPACE_BYTES, buf, NULL), Q4ADAMW_ERR_ARG);
  EXPECT(q4adamw_grad_norm(gr, 1, 5, 1.0f, NULL, 1.0f, buf + 1024, Q4ADAMW_NORM_WORKSPACE_BYTES, buf, NULL), Q4ADAMW_ERR_ARG);
  /* interchange */
  EXPECT(q4adamw_quantize(buf, 0, 0, codes, scales, NULL), 0);
  EXPECT(q4adamw_quantize(buf, 10, 2, codes, scales, NULL), Q4ADAMW_ERR_ARG);
  EXPECT(q4adamw_quantize(NULL, 10, 0, codes, scales, NULL), Q4ADAMW_ERR_ARG);
  EXPECT(q4adamw_quantize((float *)((char *)buf + 2), 10, 0, codes, scales, NULL), Q4ADAMW_ERR_ALIGN);
  EXPECT(q4adamw_dequantize(codes, scales, -3, 0, buf, NULL), Q4ADAMW_ERR_ARG);
  EXPECT(q4adamw_dequantize(codes, scales, 10, 0, NULL, NULL), Q4ADAMW_ERR_ARG);
  EXPECT(q4adamw_dequantize(codes, scales, INT64_MAX, 1, buf, NULL), Q4ADAMW_ERR_TOO_LARGE);
  free(buf);
}

static void oracle_on_ragged_sizes(void) {
  const int64_t sizes[] = {1, 127, 128, 129, 255, 1000, 4097};
  for (size_t k = 0; k < sizeof sizes / sizeof sizes[0]; ++k) {
    const int64_t n = sizes[k], nbytes = (n + 1) / 2, nblk = (n + 127) / 128;
    for (int p_dtype = 0; p_dtype < 2; ++p_dtype) {
      /* exact-size allocations: an access past the end is a finding */
      void *p = calloc((size_t)n, p_dtype ? 2 : 4);
      uint16_t *g = malloc((size_t)n * 2);
      uint8_t *m = calloc((size_t)nbytes, 1), *v = calloc((size_t)nbytes, 1);
      float *sm = calloc((size_t)nblk, 4), *sv = calloc((size_t)nblk, 4);
      float *fm = calloc((size_t)n, 4), *fv = calloc((size_t)n, 4), *back = malloc((size_t)n * 4);
      for (int64_t i = 0; i < n; ++i) g[i] = (uint16_t)((i % 7 == 0) ? 0 : (0x3a00 + (i * 37) % 512) | ((i & 1) << 15));
      if (n > 256) memset(g + 128, 0, 256);   /* an all-zero block */
      for (int step = 1; step <= 3; ++step) {
        q4o_step_quant(p, g, m, v, sm, sv, n, p_dtype, 1, B1, B2, LR, WD, EPS, (float)step);
        q4o_step_unquant(p, g, fm, fv, n, p_dtype, 1, B1, B2, LR, WD, EPS, (float)step);
      }
      for (int which = 0; which < 2; ++which) {
        q4o_dequant(which ? v : m, which ? sv : sm, n, which, back);
        q4o_quant(back, n, which, which ? v : m, which ? sv : sm);
      }
      free(p); free(g); free(m); free(v); free(sm); free(sv); free(fm); free(fv); free(back);
    }
  }
}

int main(void) {
  host_only_entry_points();
  refusals();
  oracle_on_ragged_sizes();
  printf("host_sanitize: ok\n");
  return 0;
}
