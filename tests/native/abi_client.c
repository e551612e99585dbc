/*
 * A plain C11 client of the C ABI in include/q4adamw.h: no Python, no torch, device
 * memory from hipMalloc, the null stream.  It plays the part of the reference's
 * extension glue (optim/cuda_fused_interface.cc:19-39, :49-64) for a caller that is
 * not Python, and checks every result against the scalar C oracle (test
 * infrastructure, linked here as the checker only):
 *   - packed codes and block scales bit for bit, parameters within 1e-6 relative
 *     (fp32) or one ulp of bf16 / fp16, over three steps on an odd-sized tensor, all nine
 *     pairs of parameter and gradient types
 *   - the multi-tensor entry point with an empty tensor in the list
 *   - the non-quantized entry point
 *   - quantize / dequantize against the oracle's
 *   - error codes and messages for bad arguments (nothing is launched for those)
 * Exit status 0 and a last line "abi_client: all checks passed" mean success.
 *
 * Build (tests/test_abi_client.py does this, into a temporary directory):
 *   gcc -std=c11 -O1 -D__HIP_PLATFORM_AMD__ -Iinclude -I/opt/rocm/include \
 *       tests/native/abi_client.c quantfour_adamw_cuda_amd/csrc/libq4adamw.so \
 *       oracle/libq4oracle.so -L/opt/rocm/lib -lamdhip64 -lm -o abi_client
 */
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "q4adamw.h"

/* the checker (oracle/q4_oracle.c) */
void q4o_step_quant(void *p, const void *g, uint8_t *m_codes, uint8_t *v_codes, float *m_scale,
                    float *v_scale, int64_t numel, int p_dtype, int g_dtype, float beta1,
                    float beta2, float lr, float weight_decay, float eps, float step);
void q4o_step_unquant(void *p, const void *g, float *m, float *v, int64_t numel, int p_dtype,
                      int g_dtype, float beta1, float beta2, float lr, float weight_decay,
                      float eps, float step);
void q4o_quant(const float *x, int64_t numel, int which, uint8_t *codes, float *scale);
void q4o_dequant(const uint8_t *codes, const float *scale, int64_t numel, int which, float *out);
void q4o_tables(int which, float *qmap16, float *qmid15);
float q4o_f16_to_f32(uint16_t h);
uint16_t q4o_f32_to_f16(float f);

static const float B1 = 0.9f, B2 = 0.999f, LR = 1e-3f, WD = 0.01f, EPS = 1e-8f;

#define HIP_OK(call)                                                                 \
  do {                                                                               \
    hipError_t e_ = (call);                                                          \
    if (e_ != hipSuccess) {                                                          \
      fprintf(stderr, "%s:%d %s: %s\n", __FILE__, __LINE__, #call, hipGetErrorString(e_)); \
      exit(2);                                                                       \
    }                                                                                \
  } while (0)

#define CHECK(cond, ...)                                  \
  do {                                                    \
    if (!(cond)) {                                        \
      fprintf(stderr, "%s:%d FAILED: ", __FILE__, __LINE__); \
      fprintf(stderr, __VA_ARGS__);                       \
      fprintf(stderr, "\n");                              \
      exit(1);                                            \
    }                                                     \
  } while (0)

#define Q4_OK(call)                                                     \
  do {                                                                  \
    int rc_ = (call);                                                   \
    CHECK(rc_ == 0, "%s returned %d: %s", #call, rc_, q4adamw_last_error()); \
  } while (0)

/* xorshift64* and a sum of uniforms: any fixed, portable stream of roughly normal numbers */
static uint64_t rng_state = 0x9E3779B97F4A7C15ull;
static double uniform01(void) {
  rng_state ^= rng_state >> 12;
  rng_state ^= rng_state << 25;
  rng_state ^= rng_state >> 27;
  return (double)((rng_state * 0x2545F4914F6CDD1Dull) >> 11) / 9007199254740992.0;
}
static float normalish(float sigma) {
  double s = 0.0;
  for (int i = 0; i < 12; ++i) s += uniform01();
  return (float)((s - 6.0) * sigma);
}

static uint16_t to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

static size_t elem_size(int dtype) { return dtype == Q4ADAMW_FP32 ? 4 : 2; }

static void fill(void *dst, int dtype, int64_t n, float sigma) {
  for (int64_t i = 0; i < n; ++i) {
    const float x = normalish(sigma);
    if (dtype == Q4ADAMW_BF16) ((uint16_t *)dst)[i] = to_bf16(x);
    else if (dtype == Q4ADAMW_FP16) ((uint16_t *)dst)[i] = q4o_f32_to_f16(x);
    else ((float *)dst)[i] = x;
  }
}

static float from_bf16(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static float from_16(int dtype, uint16_t h) { return dtype == Q4ADAMW_BF16 ? from_bf16(h) : q4o_f16_to_f32(h); }

/* parameters: 1e-6 relative to max(|p|, |step taken|) in fp32; in bf16 and fp16 one ulp of the
 * type on that same scale (a parameter that cancels against its update lands near zero, where
 * its own ulp is tiny) */
static void check_params(const void *dev, const void *ref, const void *before, int dtype, int64_t n,
                         const char *what) {
  for (int64_t i = 0; i < n; ++i) {
    if (dtype != Q4ADAMW_FP32) {
      const uint16_t ab = ((const uint16_t *)dev)[i], bb = ((const uint16_t *)ref)[i];
      const float a = from_16(dtype, ab), b = from_16(dtype, bb), p0 = from_16(dtype, ((const uint16_t *)before)[i]);
      const float scale = fmaxf(fmaxf(fabsf(b), fabsf(b - p0)), 1.17549435e-38f);
      const int mant = dtype == Q4ADAMW_BF16 ? 7 : 10;
      float ulp = ldexpf(1.0f, (int)floorf(log2f(scale)) - mant);
      if (dtype == Q4ADAMW_FP16) ulp = fmaxf(ulp, 5.9604644775390625e-08f);   /* fp16 subnormal spacing */
      CHECK(fabsf(a - b) <= ulp, "%s: 16-bit parameter %lld differs by more than one ulp (%04x vs %04x)", what,
            (long long)i, ab, bb);
    } else {
      const float a = ((const float *)dev)[i], b = ((const float *)ref)[i], p0 = ((const float *)before)[i];
      const float scale = fmaxf(fabsf(b), fabsf(b - p0));
      CHECK(fabsf(a - b) <= 1e-6f * scale + 1e-30f, "%s: parameter %lld: %.9g vs %.9g", what, (long long)i,
            (double)a, (double)b);
    }
  }
}

static void *dev_copy(const void *host, size_t bytes) {
  void *d = NULL;
  HIP_OK(hipMalloc(&d, bytes ? bytes : 16));
  if (bytes) HIP_OK(hipMemcpy(d, host, bytes, hipMemcpyHostToDevice));
  return d;
}

static void quantized_steps(int p_dtype, int g_dtype, int64_t n) {
  char what[64];
  snprintf(what, sizeof what, "fused_4bit p=%d g=%d n=%lld", p_dtype, g_dtype, (long long)n);
  const int64_t nbytes = (n + 1) / 2, nblk = (n + Q4ADAMW_BLOCK - 1) / Q4ADAMW_BLOCK;
  const size_t pb = (size_t)n * elem_size(p_dtype), gb = (size_t)n * elem_size(g_dtype);
  void *p = malloc(pb), *p_before = malloc(pb), *p_dev_host = malloc(pb), *g = malloc(gb);
  uint8_t *m = calloc((size_t)nbytes, 1), *v = calloc((size_t)nbytes, 1);
  float *sm = calloc((size_t)nblk, 4), *sv = calloc((size_t)nblk, 4);
  uint8_t *m_out = malloc((size_t)nbytes), *v_out = malloc((size_t)nbytes);
  float *sm_out = malloc((size_t)nblk * 4), *sv_out = malloc((size_t)nblk * 4);
  fill(p, p_dtype, n, 0.02f);
  void *dp = dev_copy(p, pb), *dg = dev_copy(NULL, 0);
  HIP_OK(hipFree(dg));
  HIP_OK(hipMalloc(&dg, gb));
  uint8_t *dm = dev_copy(m, (size_t)nbytes), *dv = dev_copy(v, (size_t)nbytes);
  float *dsm = dev_copy(sm, (size_t)nblk * 4), *dsv = dev_copy(sv, (size_t)nblk * 4);
  for (int step = 1; step <= 3; ++step) {
    fill(g, g_dtype, n, 1e-3f);
    HIP_OK(hipMemcpy(dg, g, gb, hipMemcpyHostToDevice));
    Q4_OK(q4adamw_fused_4bit(dp, dg, dm, dv, dsm, dsv, n, p_dtype, g_dtype, B1, B2, LR, WD, EPS,
                             (float)step, NULL));
    HIP_OK(hipDeviceSynchronize());
    memcpy(p_before, p, pb);
    q4o_step_quant(p, g, m, v, sm, sv, n, p_dtype, g_dtype, B1, B2, LR, WD, EPS, (float)step);
    HIP_OK(hipMemcpy(p_dev_host, dp, pb, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(m_out, dm, (size_t)nbytes, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(v_out, dv, (size_t)nbytes, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(sm_out, dsm, (size_t)nblk * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(sv_out, dsv, (size_t)nblk * 4, hipMemcpyDeviceToHost));
    CHECK(memcmp(m_out, m, (size_t)nbytes) == 0, "%s step %d: first-moment codes differ", what, step);
    CHECK(memcmp(v_out, v, (size_t)nbytes) == 0, "%s step %d: second-moment codes differ", what, step);
    CHECK(memcmp(sm_out, sm, (size_t)nblk * 4) == 0, "%s step %d: first-moment scales differ", what, step);
    CHECK(memcmp(sv_out, sv, (size_t)nblk * 4) == 0, "%s step %d: second-moment scales differ", what, step);
    check_params(p_dev_host, p, p_before, p_dtype, n, what);
    memcpy(p, p_dev_host, pb); /* the next step starts from the device's parameters */
  }
  HIP_OK(hipFree(dp)); HIP_OK(hipFree(dg)); HIP_OK(hipFree(dm)); HIP_OK(hipFree(dv));
  HIP_OK(hipFree(dsm)); HIP_OK(hipFree(dsv));
  free(p); free(p_before); free(p_dev_host); free(g); free(m); free(v); free(sm); free(sv);
  free(m_out); free(v_out); free(sm_out); free(sv_out);
  printf("ok  %s\n", what);
}

static void multi_and_small(void) {
  /* three descriptors, the middle one empty; then the non-quantized entry point */
  const int64_t sizes[3] = {70001, 0, 128 * 33};
  q4adamw_tensor t[3];
  void *hp[3], *hg[3];
  uint8_t *hm[3], *hv[3];
  float *hsm[3], *hsv[3];
  memset(t, 0, sizeof t);
  for (int i = 0; i < 3; ++i) {
    const int64_t n = sizes[i], nbytes = (n + 1) / 2, nblk = (n + 127) / 128;
    hp[i] = malloc((size_t)n * 4 + 4); hg[i] = malloc((size_t)n * 4 + 4);
    hm[i] = calloc((size_t)nbytes + 1, 1); hv[i] = calloc((size_t)nbytes + 1, 1);
    hsm[i] = calloc((size_t)nblk + 1, 4); hsv[i] = calloc((size_t)nblk + 1, 4);
    fill(hp[i], Q4ADAMW_FP32, n, 0.02f);
    fill(hg[i], Q4ADAMW_FP32, n, 1e-3f);
    t[i].numel = n;
    if (n == 0) continue;
    t[i].p = dev_copy(hp[i], (size_t)n * 4);
    t[i].g = dev_copy(hg[i], (size_t)n * 4);
    t[i].exp_avg = dev_copy(hm[i], (size_t)nbytes);
    t[i].exp_avg_sq = dev_copy(hv[i], (size_t)nbytes);
    t[i].exp_avg_scale = dev_copy(hsm[i], (size_t)nblk * 4);
    t[i].exp_avg_sq_scale = dev_copy(hsv[i], (size_t)nblk * 4);
  }
  Q4_OK(q4adamw_fused_4bit_multi(t, 3, Q4ADAMW_FP32, Q4ADAMW_FP32, B1, B2, LR, WD, EPS, 1.0f, NULL));
  HIP_OK(hipDeviceSynchronize());
  for (int i = 0; i < 3; ++i) {
    const int64_t n = sizes[i], nbytes = (n + 1) / 2, nblk = (n + 127) / 128;
    if (n == 0) continue;
    void *before = malloc((size_t)n * 4);
    memcpy(before, hp[i], (size_t)n * 4);
    q4o_step_quant(hp[i], hg[i], hm[i], hv[i], hsm[i], hsv[i], n, 0, 0, B1, B2, LR, WD, EPS, 1.0f);
    uint8_t *cm = malloc((size_t)nbytes), *cv = malloc((size_t)nbytes);
    float *csm = malloc((size_t)nblk * 4), *csv = malloc((size_t)nblk * 4), *cp = malloc((size_t)n * 4);
    HIP_OK(hipMemcpy(cm, t[i].exp_avg, (size_t)nbytes, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(cv, t[i].exp_avg_sq, (size_t)nbytes, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(csm, t[i].exp_avg_scale, (size_t)nblk * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(csv, t[i].exp_avg_sq_scale, (size_t)nblk * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(cp, t[i].p, (size_t)n * 4, hipMemcpyDeviceToHost));
    CHECK(memcmp(cm, hm[i], (size_t)nbytes) == 0 && memcmp(cv, hv[i], (size_t)nbytes) == 0,
          "multi: codes of tensor %d differ", i);
    CHECK(memcmp(csm, hsm[i], (size_t)nblk * 4) == 0 && memcmp(csv, hsv[i], (size_t)nblk * 4) == 0,
          "multi: scales of tensor %d differ", i);
    check_params(cp, hp[i], before, Q4ADAMW_FP32, n, "multi");
    free(before); free(cm); free(cv); free(csm); free(csv); free(cp);
    HIP_OK(hipFree(t[i].p)); HIP_OK(hipFree((void *)t[i].g)); HIP_OK(hipFree(t[i].exp_avg));
    HIP_OK(hipFree(t[i].exp_avg_sq)); HIP_OK(hipFree(t[i].exp_avg_scale)); HIP_OK(hipFree(t[i].exp_avg_sq_scale));
  }
  for (int i = 0; i < 3; ++i) { free(hp[i]); free(hg[i]); free(hm[i]); free(hv[i]); free(hsm[i]); free(hsv[i]); }
  printf("ok  fused_4bit_multi with an empty tensor\n");

  const int64_t n = 4096;
  float *p = malloc((size_t)n * 4), *before = malloc((size_t)n * 4), *g = malloc((size_t)n * 4);
  float *m = calloc((size_t)n, 4), *v = calloc((size_t)n, 4), *out = malloc((size_t)n * 4);
  fill(p, 0, n, 0.05f);
  fill(g, 0, n, 1e-3f);
  float *dp = dev_copy(p, (size_t)n * 4), *dg = dev_copy(g, (size_t)n * 4);
  float *dm = dev_copy(m, (size_t)n * 4), *dv = dev_copy(v, (size_t)n * 4);
  for (int step = 1; step <= 2; ++step) {
    Q4_OK(q4adamw_fused_single_tensor(dp, dg, dm, dv, n, 0, 0, B1, B2, LR, WD, EPS, (float)step, NULL));
    HIP_OK(hipDeviceSynchronize());
    memcpy(before, p, (size_t)n * 4);
    q4o_step_unquant(p, g, m, v, n, 0, 0, B1, B2, LR, WD, EPS, (float)step);
    HIP_OK(hipMemcpy(out, dm, (size_t)n * 4, hipMemcpyDeviceToHost));
    CHECK(memcmp(out, m, (size_t)n * 4) == 0, "single_tensor step %d: first moment differs", step);
    HIP_OK(hipMemcpy(out, dv, (size_t)n * 4, hipMemcpyDeviceToHost));
    CHECK(memcmp(out, v, (size_t)n * 4) == 0, "single_tensor step %d: second moment differs", step);
    HIP_OK(hipMemcpy(out, dp, (size_t)n * 4, hipMemcpyDeviceToHost));
    check_params(out, p, before, 0, n, "single_tensor");
    memcpy(p, out, (size_t)n * 4);
  }
  HIP_OK(hipFree(dp)); HIP_OK(hipFree(dg)); HIP_OK(hipFree(dm)); HIP_OK(hipFree(dv));
  free(p); free(before); free(g); free(m); free(v); free(out);
  printf("ok  fused_single_tensor\n");
}

static void interchange(void) {
  const int64_t n = 100003, nbytes = (n + 1) / 2, nblk = (n + 127) / 128;
  float *x = malloc((size_t)n * 4), *back = malloc((size_t)n * 4), *ref_back = malloc((size_t)n * 4);
  uint8_t *codes = malloc((size_t)nbytes), *ref_codes = calloc((size_t)nbytes, 1);
  float *scales = malloc((size_t)nblk * 4), *ref_scales = calloc((size_t)nblk, 4);
  for (int which = 0; which < 2; ++which) {
    fill(x, 0, n, 0.01f);
    if (which) for (int64_t i = 0; i < n; ++i) x[i] = x[i] * x[i];
    float *dx = dev_copy(x, (size_t)n * 4), *dout = dev_copy(x, (size_t)n * 4);
    uint8_t *dc = dev_copy(codes, (size_t)nbytes);
    float *ds = dev_copy(scales, (size_t)nblk * 4);
    Q4_OK(q4adamw_quantize(dx, n, which, dc, ds, NULL));
    Q4_OK(q4adamw_dequantize(dc, ds, n, which, dout, NULL));
    HIP_OK(hipDeviceSynchronize());
    HIP_OK(hipMemcpy(codes, dc, (size_t)nbytes, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(scales, ds, (size_t)nblk * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(back, dout, (size_t)n * 4, hipMemcpyDeviceToHost));
    q4o_quant(x, n, which, ref_codes, ref_scales);
    q4o_dequant(ref_codes, ref_scales, n, which, ref_back);
    CHECK(memcmp(codes, ref_codes, (size_t)nbytes) == 0, "quantize(which=%d): codes differ", which);
    CHECK(memcmp(scales, ref_scales, (size_t)nblk * 4) == 0, "quantize(which=%d): scales differ", which);
    CHECK(memcmp(back, ref_back, (size_t)n * 4) == 0, "dequantize(which=%d) differs", which);
    HIP_OK(hipFree(dx)); HIP_OK(hipFree(dout)); HIP_OK(hipFree(dc)); HIP_OK(hipFree(ds));
  }
  free(x); free(back); free(ref_back); free(codes); free(ref_codes); free(scales); free(ref_scales);
  printf("ok  quantize / dequantize\n");
}

static void tables_and_errors(void) {
  CHECK(q4adamw_version() >= 1000, "version %d", q4adamw_version());
  for (int which = 0; which < 2; ++which) {
    float a[16], am[15], b[16], bm[15];
    q4adamw_tables(which, a, am);
    q4o_tables(which, b, bm);
    CHECK(memcmp(a, b, sizeof a) == 0 && memcmp(am, bm, sizeof am) == 0, "tables(which=%d) differ", which);
  }
  float *d = NULL;
  HIP_OK(hipMalloc((void **)&d, 1 << 16));
  uint8_t *c = (uint8_t *)d + 32768;
  float *s = d + 12000;
  /* every refusal must come before anything is launched and must leave a message */
  int rc = q4adamw_fused_4bit((float *)((char *)d + 2), d + 2048, c, c + 2048, s, s + 64, 1000, 0, 0, B1, B2, LR, WD, EPS, 1.0f, NULL);
  CHECK(rc == Q4ADAMW_ERR_ALIGN && strlen(q4adamw_last_error()) > 0, "misaligned p: rc %d", rc);
  rc = q4adamw_fused_4bit(d, d + 2048, c, c + 2048, s, s + 64, 1000, 7, 0, B1, B2, LR, WD, EPS, 1.0f, NULL);
  CHECK(rc == Q4ADAMW_ERR_ARG && strlen(q4adamw_last_error()) > 0, "bad dtype tag: rc %d", rc);
  rc = q4adamw_fused_4bit(d, d + 2048, c, c + 2048, s, s + 64, 1000, 0, 0, B1, B2, -1.0f, WD, EPS, 1.0f, NULL);
  CHECK(rc == Q4ADAMW_ERR_HYPER && strlen(q4adamw_last_error()) > 0, "negative lr: rc %d", rc);
  rc = q4adamw_fused_4bit(d, d + 2048, c, c + 2048, s, s + 64, 1000, 0, 0, B1, B2, LR, WD, EPS, 0.0f, NULL);
  CHECK(rc == Q4ADAMW_ERR_HYPER, "step 0: rc %d", rc);
  rc = q4adamw_fused_4bit(d, NULL, c, c + 2048, s, s + 64, 1000, 0, 0, B1, B2, LR, WD, EPS, 1.0f, NULL);
  CHECK(rc == Q4ADAMW_ERR_ARG, "null gradient: rc %d", rc);
  rc = q4adamw_fused_4bit(d, d + 2048, c, c + 2048, s, s + 64, -5, 0, 0, B1, B2, LR, WD, EPS, 1.0f, NULL);
  CHECK(rc == Q4ADAMW_ERR_ARG, "negative numel: rc %d", rc);
  Q4_OK(q4adamw_fused_4bit(d, d + 2048, c, c + 2048, s, s + 64, 0, 0, 0, B1, B2, LR, WD, EPS, 1.0f, NULL));
  HIP_OK(hipDeviceSynchronize());
  HIP_OK(hipFree(d));
  CHECK(q4adamw_release() == 0, "release");
  printf("ok  tables, error codes\n");
}

int main(void) {
  int ndev = 0;
  HIP_OK(hipGetDeviceCount(&ndev));
  CHECK(ndev > 0, "no GPU");
  HIP_OK(hipSetDevice(0));
  tables_and_errors();
  for (int p_dtype = 0; p_dtype < 3; ++p_dtype)
    for (int g_dtype = 0; g_dtype < 3; ++g_dtype) quantized_steps(p_dtype, g_dtype, 1000003);
  quantized_steps(Q4ADAMW_FP32, Q4ADAMW_FP32, 129);
  multi_and_small();
  interchange();
  printf("abi_client: all checks passed\n");
  return 0;
}
