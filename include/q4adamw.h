/*
 * q4adamw -- C ABI of the MI355X (gfx950) fused 4-bit AdamW step.
 *
 * One shared library, plain pointers and sizes, no torch or pybind11 types.  The
 * entry points stand where the reference's pybind11 module `quantfour_cuda`
 * stands (optim/cuda_fused_interface.cc:66-69): same argument roles, same order
 * (param, grad, first moment, second moment, first-moment scales, second-moment
 * scales, beta1, beta2, lr, weight_decay, eps, step), every hyper-parameter an
 * fp32 value as pybind11 narrows them there.  Differences that a C ABI forces:
 * element count and dtypes are explicit, the HIP stream is explicit, and the
 * status comes back as an int instead of a C++ exception.
 *
 * All device pointers are borrowed for the duration of the call; tensors are
 * updated in place; nothing is retained: tensor descriptors travel in kernel
 * arguments and the library allocates no device or pinned memory.  Calls are
 * asynchronous with respect to the host: work is enqueued on `stream` (a
 * hipStream_t; NULL is the default stream).
 *
 * Return value: 0 on success, negative for an argument error, positive for a
 * hipError_t raised by the runtime.  q4adamw_last_error() describes the last
 * failure on the calling thread.
 */
#ifndef Q4ADAMW_H
#define Q4ADAMW_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element types of parameters and gradients (p_dtype, g_dtype), in any combination.
 * The reference dispatches on the parameter's type over double, float and half
 * (AT_DISPATCH_FLOATING_TYPES_AND_HALF, optim/cuda_adamw_kernels.cu:443) and takes the
 * gradient to have the same type; float and half are here, bfloat16 is added, and the
 * arithmetic is fp32 whatever the storage type.  double is not taken: there is no tag for
 * it and any other tag is refused with Q4ADAMW_ERR_ARG (a double tensor's optimizer state
 * in 4 bits has no use; callers keep fp32 master parameters instead). */
#define Q4ADAMW_FP32 0
#define Q4ADAMW_BF16 1
#define Q4ADAMW_FP16 2

#define Q4ADAMW_BLOCK 128 /* elements per quantization block (one scale each) */

#define Q4ADAMW_ERR_ARG (-1)       /* null pointer, negative size, bad dtype tag */
#define Q4ADAMW_ERR_ALIGN (-2)     /* pointer not aligned as its buffer requires */
#define Q4ADAMW_ERR_HYPER (-3)     /* hyper-parameter outside its domain         */
#define Q4ADAMW_ERR_TOO_LARGE (-4) /* a tensor beyond 2^31 - 16 chunks (2^35 elements for rank-1) */

/*
 * One quantized tensor.  Field order follows the tensor arguments of
 * fused_4bit (optim/cuda_fused_interface.cc:19-21).
 *   p             numel elements, fp32, bf16 or fp16
 *   g             numel elements, fp32, bf16 or fp16
 *   exp_avg       (numel+1)/2 bytes; byte i = code(2i) | code(2i+1) << 4
 *   exp_avg_sq    same layout
 *   exp_avg_scale ceil(numel/128) fp32 block scales of exp_avg
 *   exp_avg_sq_scale  same for exp_avg_sq
 * p and g need the alignment of their element type only, like the reference's element-wise
 * accesses (optim/cuda_adamw_kernels.cu:334-351), so views at any offset into a flat buffer
 * are taken.  16-byte aligned addresses are the fast case: a parameter tensor that is not
 * takes 6 to 9 % longer (its waves' stores share lines), a gradient tensor costs nothing
 * extra.  Code and scale buffers must be 4-byte aligned (2 bytes suffice for the codes of
 * an fp32 parameter).
 */
typedef struct q4adamw_tensor {
  void *p;
  const void *g;
  uint8_t *exp_avg;
  uint8_t *exp_avg_sq;
  float *exp_avg_scale;
  float *exp_avg_sq_scale;
  int64_t numel;
} q4adamw_tensor;

/*
 * One non-quantized tensor (fp32 moments), fields in the order of the tensor
 * arguments of fused_single_tensor (optim/cuda_fused_interface.cc:49-53).
 */
typedef struct q4adamw_small_tensor {
  void *p;
  const void *g;
  float *exp_avg;
  float *exp_avg_sq;
  int64_t numel;
} q4adamw_small_tensor;

/*
 * What a step does to the gradients besides reading them.  The reference's caller
 * pattern (tests/driver.py:53-59: zero_grad, backward, step) leaves loss-scale
 * removal, clipping and zeroing to separate passes over the gradients; the `_ex`
 * entry points fold them into the step's single read of g.
 *   grad_scale       every gradient element is multiplied by
 *   grad_scale_dev     s = grad_scale * (grad_scale_dev ? *grad_scale_dev : 1)
 *                    in fp32 (one rounded multiplication per element) before the
 *                    step uses it.  grad_scale_dev is a device fp32 scalar (e.g.
 *                    1 / loss scale, a clip coefficient, q4adamw_grad_norm's
 *                    out3[2]) or NULL.
 *   skip_if_nonzero  device fp32 scalar or NULL: when it holds a non-zero value
 *                    (an overflow flag) the call leaves parameters and optimizer
 *                    state as they are.
 *   step_consts      device memory of Q4ADAMW_STEP_CONSTS_BYTES bytes that
 *                    q4adamw_device_step has filled, or NULL.  Not NULL: the step's
 *                    derived scalars (bias corrections, step size, weight-decay factor)
 *                    are read from there and the call's own lr, weight_decay, eps and
 *                    step only pass the range check -- for a step whose number the host
 *                    does not know, e.g. inside a captured graph.  The _sr entry points
 *                    then key their noise by the step number found there.
 *   zero_grad        non-zero: the gradients are overwritten with zeros once read
 *                    (the `g` pointers are written in that case), also by a call
 *                    that skip_if_nonzero cancels: the overflowed gradients must
 *                    not reach the next accumulation.
 *   update_form      how the quantized step computes the parameter
 *                    (optim/cuda_adamw_kernels.cu:334,351:
 *                    p * wdu - step_size * (m / (sqrtf(v) / correction2_sqrt + eps))):
 *                    Q4ADAMW_UPDATE_EXACT   those seven operations, each rounded as IEEE 754
 *                                           rounds it (nvcc's defaults for sqrtf and /): the
 *                                           parameters come out bit for bit as that expression
 *                                           gives them;
 *                    Q4ADAMW_UPDATE_FOLDED  p * wdu - m * rcp(sqrt(v) * A + B), step size and
 *                                           bias correction folded into A and B, hardware
 *                                           square root and reciprocal (one ulp each): fp32
 *                                           parameters within 1e-6 of max(|p|, |step taken|),
 *                                           16-bit parameters within one ulp of their type;
 *                    Q4ADAMW_UPDATE_AUTO    (0) exact for fp32 parameters in the block-scaled
 *                                           step with nearest rounding, where it costs under
 *                                           1 % of the step; folded for 16-bit parameters,
 *                                           stochastic rounding and rank-1 scaling, where it
 *                                           costs 5 to 10 %.
 *                    Codes and scales do not depend on it.  The non-quantized step always
 *                    computes the exact form.  Entry points without options take AUTO.
 * The device scalars are read when the kernels run, not when the call returns.
 */
#define Q4ADAMW_UPDATE_AUTO 0
#define Q4ADAMW_UPDATE_EXACT 1
#define Q4ADAMW_UPDATE_FOLDED 2

typedef struct q4adamw_grad_options {
  float grad_scale;
  int zero_grad;
  const float *grad_scale_dev;
  const float *skip_if_nonzero;
  const void *step_consts;
  int update_form;
  int reserved; /* 0 */
} q4adamw_grad_options;

/* One gradient tensor for q4adamw_grad_norm: numel elements, aligned to the element type. */
typedef struct q4adamw_grad {
  const void *g;
  int64_t numel;
} q4adamw_grad;

/*
 * Fused 4-bit AdamW step on one tensor.
 * Replaces fused_4bit (optim/cuda_fused_interface.cc:19-39) and its launcher
 * cuda_fused_4bit (optim/cuda_adamw_kernels.cu:422-469).
 */
int q4adamw_fused_4bit(void *p, const void *g, uint8_t *exp_avg, uint8_t *exp_avg_sq,
                       float *exp_avg_scale, float *exp_avg_sq_scale, int64_t numel,
                       int p_dtype, int g_dtype, float beta1, float beta2, float lr,
                       float weight_decay, float eps, float step, void *stream);

/*
 * The same step over many tensors: one launch per batch of up to 48 tensors.  All
 * tensors share dtypes, hyper-parameters and step.  `tensors` is a host array that
 * is read before the call returns.  Replaces the reference's per-parameter Python
 * loop around fused_4bit (optim/fused_quantfour.py:171-292).
 */
int q4adamw_fused_4bit_multi(const q4adamw_tensor *tensors, int count, int p_dtype,
                             int g_dtype, float beta1, float beta2, float lr,
                             float weight_decay, float eps, float step, void *stream);

/* q4adamw_fused_4bit_multi with gradient options (NULL = none). */
int q4adamw_fused_4bit_multi_ex(const q4adamw_tensor *tensors, int count, int p_dtype,
                                int g_dtype, float beta1, float beta2, float lr,
                                float weight_decay, float eps, float step,
                                const q4adamw_grad_options *opt, void *stream);

/*
 * q4adamw_fused_4bit_multi_ex with stochastic rounding in the quantizer of both
 * moments: a normalised value between two neighbouring code-book entries Q[k] and
 * Q[k+1] takes the upper one with probability (x - Q[k]) / (Q[k+1] - Q[k]) instead of
 * the nearer one; values at or beyond the ends of the code book take the end codes.
 * The rule of quantize_bsearch<STOCHASTIC> quoted at
 * optim/adamw_fourbit_triton.py:1050-1075, evaluated without its division as
 * noise * (Q[k+1] - Q[k]) < x - Q[k].  The noise of an element is a hash of its index
 * and of q4adamw_sr_tensor_salt(seed, step, salts[i]) (salts == NULL: the tensor's
 * position in the list), so a call is reproducible and two steps, tensors or seeds
 * draw different noise; the reference's optimizers agree on such a seed across ranks
 * (optim/adamw_fourbit_triton.py:163-165).  Scales stay the blocks' abs-maxima.
 */
int q4adamw_fused_4bit_multi_sr(const q4adamw_tensor *tensors, int count, const uint32_t *salts,
                                uint64_t seed, int p_dtype, int g_dtype, float beta1, float beta2,
                                float lr, float weight_decay, float eps, float step,
                                const q4adamw_grad_options *opt, void *stream);

/* Host-only: the 32-bit noise salt of one tensor in one step (for tests). */
uint32_t q4adamw_sr_tensor_salt(uint64_t seed, float step, uint32_t tensor_salt);

/*
 * One quantized matrix whose second moment is rank-1 scaled: the scale of element
 * (i, j) is min(row_max[i], col_max[j]), the maxima of the second moment over row i
 * and over column j (get_variance_tensor_statistics / compute_variance_tensor_scale,
 * optim/adamw_fourbit_triton.py:738-755; scale_type "rank1", :124).  The first moment
 * keeps its per-128 block scales.  row_max/col_max (rows and cols floats) are
 * updated by the call; row_max_next/col_max_next are state-owned scratch of the same
 * sizes that must hold zeros on entry and holds zeros again afterwards.
 * rows x cols, row-major, cols >= 2; p and g aligned to their element type (see
 * q4adamw_tensor), col_max and col_max_next 16-byte aligned, the rest 4-byte aligned.  Rows of
 * a multiple of 8 elements (and at least 16) take the tuned kernels; any other row length is
 * taken element by element (matrices of fewer than 2^32 elements), as the draft scales every
 * tensor with dim() > 1 this way (optim/adamw_fourbit_triton.py:841-846).
 *
 * Tensors of three or four dimensions (lead_dims = 2 or 3): cols is the last dimension,
 * lead_shape the others, rows their product.  Every leading dimension has its own
 * statistic, the maximum over all other dimensions (the loop over x.dim() at
 * optim/adamw_fourbit_triton.py:741-745): lead_max[j] (lead_shape[j] floats, updated by the
 * call) with scratch lead_max_next[j] (zeros on entry and afterwards).  The scale of an
 * element is the minimum over all its dimensions' statistics (:749-755); row_max then holds,
 * for every flattened row, the minimum over its leading statistics -- derived state that the
 * call keeps up to date and the caller recomputes after loading a checkpoint.  lead_dims = 0
 * or 1: a matrix, the lead_* fields are not read.
 */
typedef struct q4adamw_rank1_tensor {
  void *p;
  const void *g;
  uint8_t *exp_avg;
  uint8_t *exp_avg_sq;
  float *exp_avg_scale;
  float *row_max;
  float *col_max;
  float *row_max_next;
  float *col_max_next;
  int64_t rows;
  int64_t cols;
  int32_t lead_dims;
  int32_t reserved;
  int64_t lead_shape[3];
  float *lead_max[3];
  float *lead_max_next[3];
} q4adamw_rank1_tensor;

/*
 * The fused step with a rank-1-scaled second moment, per batch of up to 32 tensors
 * three launches: new second moments reduced to row and column maxima, the update
 * (dequantize with the old maxima, quantize with the new ones), and the commit of the
 * new maxima.  Everything else as q4adamw_fused_4bit_multi_ex (opt may be NULL).  The
 * device form of variance_quant / variance_dequant with scale_type "rank1"
 * (optim/adamw_fourbit_triton.py:498-527, :803-863) inside the fused step
 * (optim/cuda_adamw_kernels.cu:266-419).
 */
int q4adamw_fused_4bit_rank1_multi(const q4adamw_rank1_tensor *tensors, int count, int p_dtype,
                                   int g_dtype, float beta1, float beta2, float lr,
                                   float weight_decay, float eps, float step,
                                   const q4adamw_grad_options *opt, void *stream);

/*
 * q4adamw_fused_4bit_rank1_multi with stochastic rounding of both moments: the rule and
 * the noise of q4adamw_fused_4bit_multi_sr (salts, seed as there), the second moment's
 * quotient taken with its rank-1 scale min(row_max[i], col_max[j]).  The combination of
 * the draft's settings scale_type "rank1" (optim/adamw_fourbit_triton.py:124) and
 * round_type "stochastic" (:1050-1075).
 */
int q4adamw_fused_4bit_rank1_multi_sr(const q4adamw_rank1_tensor *tensors, int count,
                                      const uint32_t *salts, uint64_t seed, int p_dtype, int g_dtype,
                                      float beta1, float beta2, float lr, float weight_decay,
                                      float eps, float step, const q4adamw_grad_options *opt,
                                      void *stream);

/*
 * Non-quantized AdamW step (fp32 moments) on one tensor.
 * Replaces fused_single_tensor (optim/cuda_fused_interface.cc:49-64) and
 * cuda_fused_single_tensor (optim/cuda_adamw_kernels.cu:136-164).
 */
int q4adamw_fused_single_tensor(void *p, const void *g, float *exp_avg, float *exp_avg_sq,
                                int64_t numel, int p_dtype, int g_dtype, float beta1,
                                float beta2, float lr, float weight_decay, float eps,
                                float step, void *stream);

/* Many non-quantized tensors, one launch per batch of up to 80 (`tensors` is a host array). */
int q4adamw_fused_single_tensor_multi(const q4adamw_small_tensor *tensors, int count,
                                      int p_dtype, int g_dtype, float beta1, float beta2,
                                      float lr, float weight_decay, float eps, float step,
                                      void *stream);

/* q4adamw_fused_single_tensor_multi with gradient options (NULL = none). */
int q4adamw_fused_single_tensor_multi_ex(const q4adamw_small_tensor *tensors, int count,
                                         int p_dtype, int g_dtype, float beta1, float beta2,
                                         float lr, float weight_decay, float eps, float step,
                                         const q4adamw_grad_options *opt, void *stream);

/*
 * Global L2 norm of a set of gradient tensors and the clip coefficient that follows
 * from it: what torch.nn.utils.clip_grad_norm_ computes before it rescales the
 * gradients (the reference's callers clip between backward and step; the rescaling
 * itself is the `_ex` entry points' multiplier).  With
 *   s = grad_scale * (grad_scale_dev ? *grad_scale_dev : 1):
 *   out3[0] = |s| * sqrt(sum g^2)               norm of the scaled gradients (fp32)
 *   out3[1] = min(1, max_norm / (out3[0] + 1e-6))   clip coefficient; 1 if max_norm <= 0
 *   out3[2] = s * out3[1]                       multiplier to hand to the step
 * Squares are summed in fp64 in a fixed order (the result does not depend on
 * scheduling).  `workspace` is device memory of Q4ADAMW_NORM_WORKSPACE_BYTES bytes,
 * 8-byte aligned, overwritten by the call; out3 is three device floats.  All tensors
 * share g_dtype.
 */
#define Q4ADAMW_NORM_WORKSPACE_BYTES 16384
int q4adamw_grad_norm(const q4adamw_grad *grads, int count, int g_dtype, float grad_scale,
                      const float *grad_scale_dev, float max_norm, void *workspace,
                      size_t workspace_bytes, float *out3, void *stream);

/*
 * q4adamw_grad_norm for callers that cannot allocate device memory and so have no workspace
 * to pass: code under graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * No counterpart in the reference.  The partial sums live in a 16 KiB (2048 x fp64) array
 * inside the library's device image, one copy per GPU, held until the process ends; the
 * call allocates and frees nothing and gives the results of q4adamw_grad_norm bit for bit.
 * That array's size does not depend on the input: the limits are q4adamw_grad_norm's own (a
 * tensor of more than 2^31 - 16 chunks of 32 KiB is refused with Q4ADAMW_ERR_TOO_LARGE), and
 * device ordinals of 64 and above are refused with Q4ADAMW_ERR_ARG.  Every partial sum is
 * overwritten before it is read, so nothing of an earlier call survives.  All calls on one
 * GPU share the one array: two calls that overlap there (different streams, different
 * threads) race; calls on one stream, or otherwise ordered, do not.  The first call on a
 * device asks the runtime for the array's address (no allocation); make it outside a capture.
 * The address is kept per device for the life of the process: the stream must belong to the
 * current device (a stream of another device is refused with Q4ADAMW_ERR_ARG), and a process
 * that resets a device (hipDeviceReset) must not call this entry point on it afterwards.
 */
int q4adamw_grad_norm_static(const q4adamw_grad *grads, int count, int g_dtype, float grad_scale,
                             const float *grad_scale_dev, float max_norm, float *out3, void *stream);

/*
 * A step whose number lives on the device.  The reference derives the scalars of a step on
 * the host from the step number it is given (optim/cuda_adamw_kernels.cu:435-440); a host
 * that replays a captured graph has no step number to give.  q4adamw_bias_table (host only)
 * tabulates the two step-dependent values, 1 - beta1^t and sqrt(1 - beta2^t), for t =
 * first_step .. first_step + count - 1, two floats per step, computed as the launcher
 * computes them; the caller copies the table to the device.  q4adamw_device_step enqueues a
 * one-thread kernel that adds 1 to the fp32 counter *step_dev (unless *skip_if_nonzero is
 * non-zero: then it changes nothing), takes the table entry of the new step number (steps
 * past the table take its last entry, so the table should reach the step at which both
 * values have become 1), takes lr from *lr_dev if lr_dev is not NULL, and writes the derived
 * scalars to consts_dev (Q4ADAMW_STEP_CONSTS_BYTES bytes, 16-byte aligned) with the host's
 * own operations: a step made with them equals, bit for bit, the step made with that step
 * number on the host.  Pass consts_dev as q4adamw_grad_options.step_consts.
 */
#define Q4ADAMW_STEP_CONSTS_BYTES 64
int q4adamw_bias_table(float beta1, float beta2, int64_t first_step, int64_t count, float *out2);
int q4adamw_device_step(float *step_dev, const float *bias_table_dev, int64_t table_first_step,
                        int64_t table_steps, const float *lr_dev, float beta1, float beta2, float lr,
                        float weight_decay, float eps, const float *skip_if_nonzero, void *consts_dev,
                        void *stream);

/*
 * Quantize one fp32 moment: per block of 128 consecutive elements the scale is the
 * abs-max, every element is divided by it and mapped to the nearest code (ties go
 * down), codes are packed two per byte.  which: 0 first moment (signed map),
 * 1 second moment (unsigned map).  codes: (numel+1)/2 bytes, scales: ceil(numel/128).
 * The device form of momentum_quant / variance_quant with per-block scaling
 * (optim/adamw_fourbit_triton.py:556-588, :618-630) and of q_mapping
 * (optim/cuda_adamw_kernels.cu:167-194); used to take over fp32 AdamW state.
 */
int q4adamw_quantize(const float *x, int64_t numel, int which, uint8_t *codes, float *scales,
                     void *stream);

/*
 * Inverse layout step: out[i] = code_book[code(i)] * scales[i / 128], fp32.  The
 * device form of the dequantize pass (optim/cuda_adamw_kernels.cu:329-343,
 * optim/adamw_fourbit_triton.py:423-450); used to hand state back as fp32.
 */
int q4adamw_dequantize(const uint8_t *codes, const float *scales, int64_t numel, int which,
                       float *out, void *stream);

/*
 * q4adamw_quantize_rank1 with the scales given instead of computed: element (i, j) is divided
 * by min(row_scale[i], col_max[j]).  For tensors of more than two dimensions, whose rows'
 * scales are the minimum over the leading dimensions' statistics (q4adamw_rank1_tensor).
 */
int q4adamw_quantize_rank1_scaled(const float *x, int64_t rows, int64_t cols, const float *row_scale,
                                  const float *col_max, uint8_t *codes, void *stream);

/*
 * The same pair for a second moment with rank-1 scaling: x is a rows x cols fp32
 * matrix; row_max[i] / col_max[j] receive the abs-maxima of
 * row i / column j, every element is divided by min(row_max[i], col_max[j]) and
 * mapped to the nearest code of the second moment's map (variance_quant_scaling and
 * variance_quant, optim/adamw_fourbit_triton.py:803-863); dequantize multiplies back
 * (:520-527).
 */
int q4adamw_quantize_rank1(const float *x, int64_t rows, int64_t cols, uint8_t *codes,
                           float *row_max, float *col_max, void *stream);
int q4adamw_dequantize_rank1(const uint8_t *codes, const float *row_max, const float *col_max,
                             int64_t rows, int64_t cols, float *out, void *stream);

/*
 * Host-only: the six fp32 scalars the launcher derives from the hyper-parameters
 * (optim/cuda_adamw_kernels.cu:435-440), in that order: correction1,
 * correction2_sqrt, step_size, weight_decay_update, resid_beta1, resid_beta2.
 */
void q4adamw_derive_scalars(float beta1, float beta2, float lr, float weight_decay,
                            float step, float *out6);

/*
 * Host-only: code books and thresholds as the kernels hold them
 * (optim/cuda_adamw_kernels.cu:25-98).  which: 0 first moment, 1 second moment.
 */
void q4adamw_tables(int which, float *qmap16, float *qmid15);

/*
 * Host-only: entry `index` (0..2047) of the first-moment bucket table, indexed by
 * the top eleven bits of a normalised value's fp32 pattern; out2[0] = lower guard
 * bound with the base code in its low nibble, out2[1] = upper guard bound (fp32
 * bit patterns).  For tests.
 */
int q4adamw_mtable_entry(uint32_t index, uint32_t *out2);

/*
 * Host-only: the fused kernel holds 256 of those entries in LDS and indexes them
 * by the high byte of the normalised value converted to half precision toward
 * zero; this returns the index (0..2047) of the entry that `half_index` (0..255)
 * stands for, or a negative status.  For tests.
 */
int q4adamw_mtable_half_bucket(uint32_t half_index);

/*
 * Host-only: the two tables the first moment's stochastic rounding indexes in its fast
 * path (no counterpart in the reference, which only quotes the rounding rule,
 * optim/adamw_fourbit_triton.py:1050-1075).  q4adamw_sr_bucket_entry: entry `half_index`
 * (0..255) of the table indexed like the one above: out2[0] = fp32 bits of the code-book
 * value inside the bucket (0x7f000000 if none), out2[1] = number of code-book values below
 * the whole bucket; k = out2[1] + (q >= value) is the number of code-book values <= q.
 * q4adamw_sr_affine_entry: entry k (0..16) of the table that turns a normalised value
 * into its code coordinate, out2 = {slope, offset}: floor(slope * q + offset - noise) is
 * the code wherever that value is clear of an integer.  For tests.
 */
int q4adamw_sr_bucket_entry(uint32_t half_index, uint32_t *out2);
int q4adamw_sr_affine_entry(uint32_t k, float *out2);

/*
 * Host-only.  A grid of the HIP runtime holds fewer than 2^32 work-items, i.e. at most
 * 2^24 - 8 workgroups of 256 threads (1.7e10 fp32 elements of the fused step), so the entry
 * points run a large batch -- or one very large tensor, e.g. a flat sharded parameter -- as
 * several grids.  q4adamw_grid_plan returns how many grids `chunks` workgroups of `threads`
 * threads take and writes the first `capacity` of them as (first chunk, number of chunks).
 * q4adamw_set_grid_limit lowers the number of workgroups per grid for the calling process
 * (0 restores the runtime's limit; values are rounded down to a multiple of 8): for tests that
 * exercise the split without 80 GB of parameters.  The reference launches one grid per tensor
 * with a 32-bit element count (optim/cuda_adamw_kernels.cu:430-432) and stops at 2^31 elements.
 */
int q4adamw_grid_plan(uint64_t chunks, int threads, uint64_t *bases, uint64_t *counts, int capacity);
/* Host-only, for tests: which of its three update kernels q4adamw_fused_4bit_rank1_multi runs on
 * a rows x cols matrix: 0 = tiles aligned to the rows, 1 = tiles anywhere in rows of at least a
 * tile, 2 = rows shorter than a tile, 3 = rows of any length (no multiple of 8, or below 16).  both_16_bit: parameters and gradients are 16-bit types
 * (tiles of 512 elements instead of 256). */
int q4adamw_rank1_form(int64_t rows, int64_t cols, int both_16_bit);
void q4adamw_set_grid_limit(uint64_t workgroups);

/*
 * Self-check of the exact parameter update (Q4ADAMW_UPDATE_EXACT) on the GPU the call runs on.
 * The exact form computes sqrtf and the two divisions of optim/cuda_adamw_kernels.cu:351 with
 * short sequences around the hardware's square-root and reciprocal estimates; one of them rests
 * on a property of the reciprocal estimate that arithmetic alone does not give for divisors whose
 * mantissa is all ones.  This call walks every fp32 pattern of the sequences' domains through
 * them on the device and adds to counts6 (six device uint64, zeroed by the caller):
 *   [0] square roots, [1] refined reciprocals, [2] quotients that differ from the correctly
 *   rounded result; [3] square roots and [4] quotients of the general expansions (taken by
 *   lanes outside the domains) that differ; [5] patterns walked (2 566 914 050).
 * [0]..[4] must come back 0; if not, pass Q4ADAMW_UPDATE_FOLDED and report the GPU.  No
 * counterpart in the reference (its sqrtf and / are nvcc's).  About a second of GPU time.
 */
int q4adamw_rounding_selfcheck(uint64_t *counts6, void *stream);

/* Kept for callers that pair an init with a release: the library holds no device
 * memory, so this does nothing and returns 0. */
int q4adamw_release(void);

/* Message for the last non-zero status returned on this thread ("" if none). */
const char *q4adamw_last_error(void);

/* ABI version: major * 1000 + minor. */
int q4adamw_version(void);

#ifdef __cplusplus
}
#endif
#endif /* Q4ADAMW_H */
