"""TEST INFRASTRUCTURE -- vectorised torch-CPU restatement of the reference's
PyTorch path for the 4-bit AdamW step.

A checker and the timed CPU baseline, not a product path: only tests/, the smoke
check and the cpu_baseline leg of bench.py import this module.

It keeps the three-pass structure of the reference's pure-PyTorch draft
(optim/adamw_fourbit_triton.py:385-495): (1) unpack + dequantize the moments into
materialised fp32 tensors, (2) AdamW update with separate torch ops, (3) per-128
abs-max, divide, quantize, pack (optim/adamw_fourbit_triton.py:618-630,
:1020-1047).  Operation order and fp32 derived scalars follow the fused CUDA path
(optim/cuda_adamw_kernels.cu:334-351, :435-440) so that this file and the scalar
C oracle (q4_oracle.c) are two independent statements of one arithmetic and must
agree bit for bit.  The reference's per-element Python binary search
(adamw_fourbit_triton.py:1002-1009) is replaced by torch.bucketize over the
midpoint table, which returns the same code for every non-NaN input.

Every torch op below rounds once to fp32; none of them takes an ``alpha``/``value``
multiplier, so no fused multiply-add hides in the update.

The functions follow the device of their inputs.  On the CPU this is the timed
baseline and the second restatement; on a GPU (plain torch element-wise kernels,
nothing of this build's HIP code) it serves as the checker at sizes the CPU cannot
finish in seconds, after the same test has checked it against the C oracle.
"""
import math

import numpy as np
import torch

BLOCK = 128

# optim/adamw_fourbit_triton.py:16-97 (same literals as cuda_adamw_kernels.cu:25-98)
_QMAP_M = [-0.8875, -0.6625, -0.4375, -0.2125, -0.0775, -0.0325, -0.0055, 0.0,
           0.0055, 0.0325, 0.0775, 0.2125, 0.4375, 0.6625, 0.8875, 1.0]
_QMID_M = [-0.775, -0.55, -0.325, -0.145, -0.055, -0.019, -0.00275, 0.00275,
           0.019, 0.055, 0.145, 0.325, 0.55, 0.775, 0.94375]
_QMAP_V = [(k + 1) / 16 for k in range(16)]
_QMID_V = [(2 * k + 1) / 32 for k in range(1, 16)]

QMAP = (torch.tensor(_QMAP_M, dtype=torch.float32), torch.tensor(_QMAP_V, dtype=torch.float32))
QMID = (torch.tensor(_QMID_M, dtype=torch.float32), torch.tensor(_QMID_V, dtype=torch.float32))


def derive_scalars(beta1, beta2, lr, weight_decay, step):
    """cuda_adamw_kernels.cu:435-440 in fp32 tensors (0-dim)."""
    f = lambda x: torch.tensor(x, dtype=torch.float32)
    one = f(1.0)
    b1, b2, lr_, wd, st = f(beta1), f(beta2), f(lr), f(weight_decay), f(float(step))
    # powf as a double-precision pow rounded once to fp32 (torch.pow on fp32 tensors
    # is a vectorised approximation that differs from libm's powf in the last bit)
    pw1 = f(math.pow(b1.item(), float(step)))
    pw2 = f(math.pow(b2.item(), float(step)))
    c1 = one - pw1
    c2s = f(math.sqrt((one - pw2).item()))
    return dict(c1=c1, c2s=c2s, ss=lr_ / c1, wdu=one - lr_ * wd, r1=one - b1, r2=one - b2,
                b1=b1, b2=b2)


def unpack(codes, numel):
    """byte i -> elements 2i (low nibble) and 2i+1 (high nibble)."""
    lo = codes & 15
    hi = codes >> 4
    return torch.stack((lo, hi), dim=1).reshape(-1)[:numel].to(torch.int64)


def pack(q, numel):
    if numel % 2:
        q = torch.cat((q, q.new_zeros(1)))
    q = q.reshape(-1, 2).to(torch.uint8)
    return q[:, 0] | (q[:, 1] << 4)


def dequantize(codes, scale, numel, which):
    """pass 1: materialise an fp32 moment (adamw_fourbit_triton.py:423-450)."""
    idx = unpack(codes, numel)
    vals = QMAP[which].to(codes.device)[idx]
    s = scale.repeat_interleave(BLOCK)[:numel]
    return vals * s


def quantize(x, which):
    """pass 3: group abs-max, divide, nearest code, pack."""
    numel = x.numel()
    nblk = (numel + BLOCK - 1) // BLOCK
    padded = torch.zeros(nblk * BLOCK, dtype=torch.float32, device=x.device)
    padded[:numel] = x
    grouped = padded.view(nblk, BLOCK)
    # :623-624, :1078-1087; like the C oracle's running maximum, a NaN never becomes the scale
    max1 = torch.nan_to_num(grouped.abs(), nan=0.0, posinf=float("inf")).amax(dim=1, keepdim=True)
    qx = grouped.div(max1)                                   # :625 (0/0 -> NaN)
    # number of midpoints strictly below x; NaN must land on 0
    q = torch.bucketize(torch.nan_to_num(qx, nan=-2.0), QMID[which].to(x.device), right=False)
    return pack(q.reshape(-1)[:numel], numel), max1.reshape(-1)


def adamw_update(p, g, m, v, sc, eps):
    """pass 2: cuda_adamw_kernels.cu:334-351 with separate, individually rounded ops."""
    sc = {k: t.to(p.device) for k, t in sc.items()}
    m_new = sc["b1"] * m + sc["r1"] * g
    v_new = sc["b2"] * v + sc["r2"] * (g * g)
    if v_new.is_cuda:
        root = torch.sqrt(v_new)        # feeds only the parameters (tolerance class)
    else:
        # torch.sqrt on CPU fp32 is not correctly rounded in every lane; numpy's is
        root = torch.from_numpy(np.sqrt(v_new.numpy()))
    denom = root / sc["c2s"] + torch.tensor(eps, dtype=torch.float32, device=p.device)
    p_new = p * sc["wdu"] - sc["ss"] * (m_new / denom)
    return p_new, m_new, v_new


def step_quant(p, g, m_codes, v_codes, m_scale, v_scale, *, beta1, beta2, lr,
               weight_decay, eps, step):
    """Returns new (p, m_codes, v_codes, m_scale, v_scale); p keeps its dtype."""
    numel = p.numel()
    sc = derive_scalars(beta1, beta2, lr, weight_decay, step)
    m = dequantize(m_codes, m_scale, numel, 0)
    v = dequantize(v_codes, v_scale, numel, 1)
    p_new, m_new, v_new = adamw_update(p.reshape(-1).float(), g.reshape(-1).float(), m, v, sc, eps)
    mc, ms = quantize(m_new, 0)
    vc, vs = quantize(v_new, 1)
    return p_new.to(p.dtype).view_as(p), mc, vc, ms, vs


def step_unquant(p, g, m, v, *, beta1, beta2, lr, weight_decay, eps, step):
    sc = derive_scalars(beta1, beta2, lr, weight_decay, step)
    p_new, m_new, v_new = adamw_update(p.reshape(-1).float(), g.reshape(-1).float(),
                                       m.reshape(-1), v.reshape(-1), sc, eps)
    return p_new.to(p.dtype).view_as(p), m_new, v_new


# ---------------------------------------------------------------------------
# rank-1 scaling of the second moment (2-D tensors)
#
# The reference sketches it in its PyTorch draft only: statistics = per-row and
# per-column maxima (get_variance_tensor_statistics / max_reduce_except_dim,
# optim/adamw_fourbit_triton.py:738-746, :1080-1090), scale tensor = their
# broadcast minimum (compute_variance_tensor_scale, :749-755; sqs_scale_tensor,
# :537-545), quantize x.div(scale) (:834-863), dequantize x.mul(scale) (:520-527).
# The code book stays the fused path's linear map.  The draft never runs this
# against data, so parity with the reference is UNPINNED; the functions are pinned
# by brute force on small matrices, by closed forms and by the scalar C restatement of
# the whole step (q4o_step_quant_variants in q4_oracle.c), which must give the same bits
# (tests/test_oracle_pins.py).
# ---------------------------------------------------------------------------
def rank1_scale(row_max, col_max):
    """compute_variance_tensor_scale for a matrix: min(row_max[i], col_max[j])."""
    return torch.minimum(row_max.reshape(-1, 1), col_max.reshape(1, -1))


def dequantize_rank1(codes, row_max, col_max):
    rows, cols = row_max.numel(), col_max.numel()
    idx = unpack(codes, rows * cols)
    vals = QMAP[1].to(codes.device)[idx].view(rows, cols)
    return vals * rank1_scale(row_max, col_max)


def quantize_rank1(x):
    """x: fp32 matrix (non-negative).  Returns (packed codes, row_max, col_max)."""
    ax = torch.nan_to_num(x.abs(), nan=0.0, posinf=float("inf"))   # a NaN never becomes a maximum
    row_max = ax.amax(dim=1)                                 # max over all dims except 0
    col_max = ax.amax(dim=0)                                 # max over all dims except 1
    qx = x.div(rank1_scale(row_max, col_max))                # 0/0 -> NaN -> code 0
    q = torch.bucketize(torch.nan_to_num(qx, nan=-2.0), QMID[1].to(x.device), right=False)
    return pack(q.reshape(-1), x.numel()), row_max, col_max


def step_quant_rank1(p, g, m_codes, v_codes, m_scale, row_max, col_max, *, beta1, beta2, lr,
                     weight_decay, eps, step):
    """The fused step with block-scaled first moment and rank-1-scaled second moment.
    p, g: matrices [rows, cols].  Returns new (p, m_codes, v_codes, m_scale, row_max,
    col_max)."""
    rows, cols = p.shape
    numel = p.numel()
    sc = derive_scalars(beta1, beta2, lr, weight_decay, step)
    m = dequantize(m_codes, m_scale, numel, 0)
    v = dequantize_rank1(v_codes, row_max, col_max).reshape(-1)
    p_new, m_new, v_new = adamw_update(p.reshape(-1).float(), g.reshape(-1).float(), m, v, sc, eps)
    mc, ms = quantize(m_new, 0)
    vc, rmax, cmax = quantize_rank1(v_new.view(rows, cols))
    return p_new.to(p.dtype).view_as(p), mc, vc, ms, rmax, cmax


# Tensors of more than two dimensions: one statistic per dimension, the maximum over all
# other dimensions (get_variance_tensor_statistics loops over x.dim(),
# optim/adamw_fourbit_triton.py:738-746), the scale of an element their broadcast minimum
# (compute_variance_tensor_scale, :749-755).  max_dims: one tensor per dimension in keepdim
# shape ([d0,1,1], [1,d1,1], [1,1,d2] for a 3-D tensor), as the draft's metadata holds them.
def rank1_stats_nd(x):
    ax = torch.nan_to_num(x.abs(), nan=0.0, posinf=float("inf"))   # a NaN never becomes a maximum
    out = []
    for i in range(x.dim()):
        others = [d for d in range(x.dim()) if d != i]
        out.append(ax.amax(dim=others, keepdim=True))
    return out


def rank1_scale_nd(max_dims):
    scale = max_dims[0]
    for m in max_dims[1:]:
        scale = torch.minimum(scale, m)                      # broadcasting
    return scale


def dequantize_rank1_nd(codes, max_dims):
    scale = rank1_scale_nd(max_dims)
    idx = unpack(codes, scale.numel())
    return QMAP[1].to(codes.device)[idx].view(scale.shape) * scale


def quantize_rank1_nd(x, u=None):
    """x: fp32 tensor of two or more dimensions (non-negative).  u: float32 numpy noise per
    element for stochastic rounding, or None for the nearest code.  Returns (packed codes,
    max_dims)."""
    max_dims = rank1_stats_nd(x)
    qx = x.div(rank1_scale_nd(max_dims))                     # 0/0 -> NaN -> code 0
    if u is None:
        q = torch.bucketize(torch.nan_to_num(qx, nan=-2.0), QMID[1].to(x.device), right=False).reshape(-1)
    else:
        q = torch.from_numpy(sr_codes(qx.reshape(-1).numpy(), 1, np.asarray(u, np.float32)).astype(np.int64))
    return pack(q, x.numel()), max_dims


def step_quant_rank1_nd(p, g, m_codes, v_codes, m_scale, max_dims, *, beta1, beta2, lr, weight_decay, eps,
                        step, seed=None, tensor_salt=0):
    """The fused step on a tensor of two or more dimensions with a rank-1-scaled second moment
    (with a seed: stochastic rounding of both moments).  Returns new (p, m_codes, v_codes,
    m_scale, max_dims)."""
    numel = p.numel()
    sc = derive_scalars(beta1, beta2, lr, weight_decay, step)
    m = dequantize(m_codes, m_scale, numel, 0)
    v = dequantize_rank1_nd(v_codes, max_dims).reshape(-1)
    p_new, m_new, v_new = adamw_update(p.reshape(-1).float(), g.reshape(-1).float(), m, v, sc, eps)
    if seed is None:
        mc, ms = quantize(m_new, 0)
        vc, new_dims = quantize_rank1_nd(v_new.view(p.shape))
    else:
        um, uv = sr_noise(numel, sr_tensor_salt(seed, step, tensor_salt))
        mc, ms = quantize_sr(m_new, 0, um)
        vc, new_dims = quantize_rank1_nd(v_new.view(p.shape), uv)
    return p_new.to(p.dtype).view_as(p), mc, vc, ms, new_dims


# ---------------------------------------------------------------------------
# stochastic rounding in the quantizer
#
# The reference quotes lpmm's quantizer in a docstring and never runs it
# (optim/adamw_fourbit_triton.py:969-997 kernel with Philox noise, :1050-1075
# quantize_bsearch<STOCHASTIC>): the value's interval [Q[k], Q[k+1]) of the code book is
# found, proba = (x - Q[k]) / (Q[k+1] - Q[k]), and the upper code is taken when
# rn(proba + noise - 0.5) is non-zero, i.e. with probability proba; values at or beyond the
# ends of the code book take the end codes.  This build's statement of it avoids the
# division and fixes the noise as a function of (seed, step, tensor, element), so that the
# result is reproducible bit for bit:
#     up  <=>  RN(u * w[k]) < RN(q - Q[k]),   w[k] = RN(Q[k+1] - Q[k]),
#     u = (2 n + 1) / 2^17 with n a 16-bit hash value (never 0, never 1).
# Parity with the reference is UNPINNED (it has no runnable counterpart); pinned by
# brute force, by the scalar C restatement (q4o_sr_noise, q4o_quantize_sr,
# q4o_step_quant_variants), by exactness on code-book values and by the rounding's mean
# (tests/test_oracle_pins.py).
# ---------------------------------------------------------------------------
_M32 = np.uint64(0xFFFFFFFF)


def lowbias32(x):
    """A 32-bit integer mixer (two multiply-xorshift rounds); x: numpy array of uint32
    values held in uint64."""
    x = np.asarray(x, np.uint64) & _M32
    x ^= x >> np.uint64(16)
    x = (x * np.uint64(0x7FEB352D)) & _M32
    x ^= x >> np.uint64(15)
    x = (x * np.uint64(0x846CA68B)) & _M32
    x ^= x >> np.uint64(16)
    return x


def sr_tensor_salt(seed, step, tensor_salt):
    """32-bit salt of one tensor in one step: nested mixes of the tensor's salt, the step
    number and the two halves of the 64-bit seed."""
    h = lowbias32(np.uint64(int(tensor_salt) & 0xFFFFFFFF))
    h = lowbias32(h ^ np.uint64(int(step) & 0xFFFFFFFF))
    h = lowbias32(h ^ np.uint64((int(seed) >> 32) & 0xFFFFFFFF))
    h = lowbias32(h ^ np.uint64(int(seed) & 0xFFFFFFFF))
    return int(h)


def sr_noise(numel, salt):
    """(u_first_moment, u_second_moment) for elements 0..numel-1 of a tensor: float32 arrays
    of values (2 n + 1) / 2^17, n = high / low half of the element's hash."""
    e = np.arange(numel, dtype=np.uint64)
    key = (e & _M32) ^ np.uint64(salt) ^ (((e >> np.uint64(32)) * np.uint64(0x9E3779B9)) & _M32)
    h = lowbias32(key)
    to_u = lambda n: ((2.0 * n.astype(np.float64) + 1.0) / 2.0 ** 17).astype(np.float32)   # exact
    return to_u(h >> np.uint64(16)), to_u(h & np.uint64(0xFFFF))


def quantize_sr(x, which, u):
    """Per-128 abs-max scale, then stochastic rounding between the two neighbouring code-book
    values.  x: fp32 torch vector, u: float32 numpy noise per element.  Returns (packed
    codes, scales)."""
    numel = x.numel()
    nblk = (numel + BLOCK - 1) // BLOCK
    padded = np.zeros(nblk * BLOCK, np.float32)
    padded[:numel] = x.numpy()
    noise = np.zeros(nblk * BLOCK, np.float32)
    noise[:numel] = u
    grouped = padded.reshape(nblk, BLOCK)
    max1 = np.fmax.reduce(np.abs(grouped), axis=1, initial=0.0, keepdims=True)   # a NaN never becomes the scale
    with np.errstate(invalid="ignore", divide="ignore"):
        q = (grouped / max1).reshape(-1)                     # 0/0 -> NaN -> code 0
    code = sr_codes(q, which, noise)
    return pack(torch.from_numpy(code.astype(np.int64))[:numel], numel), torch.from_numpy(max1.reshape(-1))


def sr_codes(q, which, noise):
    """Stochastic rounding of normalised values q (float32 numpy, NaN -> code 0) with one
    noise value per element: numpy int codes."""
    Q = QMAP[which].numpy()
    # k_raw = number of code-book values <= q; the tables are extended so that both ends
    # need no special case: below Q[0] the "gap" is 0 (always up, from -1 to 0), at or
    # above Q[15] it is infinite (never up)
    k_raw = np.searchsorted(Q, np.nan_to_num(q, nan=-4.0), side="right")
    lower = np.concatenate(([-np.finfo(np.float32).max], Q)).astype(np.float32)
    gap = np.concatenate(([0.0], (Q[1:] - Q[:-1]).astype(np.float32), [np.inf])).astype(np.float32)
    with np.errstate(invalid="ignore", over="ignore"):
        d = q - lower[k_raw]
        t = noise * gap[k_raw]
        up = t < d
    code = np.clip(k_raw - 1 + up, 0, 15)
    code[np.isnan(q)] = 0
    return code


def quantize_rank1_sr(x, u):
    """quantize_rank1 with stochastic rounding: x fp32 matrix (CPU), u float32 numpy noise per
    element (row-major).  Returns (packed codes, row maxima, column maxima)."""
    ax = torch.nan_to_num(x.abs(), nan=0.0, posinf=float("inf"))   # statistics as in quantize_rank1
    row_max = ax.amax(dim=1)
    col_max = ax.amax(dim=0)
    q = x.div(rank1_scale(row_max, col_max)).reshape(-1).numpy()   # 0/0 -> NaN -> code 0
    code = sr_codes(q, 1, np.asarray(u, np.float32))
    return pack(torch.from_numpy(code.astype(np.int64)), x.numel()), row_max, col_max


def step_quant_rank1_sr(p, g, m_codes, v_codes, m_scale, row_max, col_max, *, seed, tensor_salt, beta1,
                        beta2, lr, weight_decay, eps, step):
    """step_quant_rank1 with stochastic rounding of both moments (CPU tensors): the first
    moment as in step_quant_sr, the second moment's quotient taken with its rank-1 scale."""
    rows, cols = p.shape
    numel = p.numel()
    sc = derive_scalars(beta1, beta2, lr, weight_decay, step)
    m = dequantize(m_codes, m_scale, numel, 0)
    v = dequantize_rank1(v_codes, row_max, col_max).reshape(-1)
    p_new, m_new, v_new = adamw_update(p.reshape(-1).float(), g.reshape(-1).float(), m, v, sc, eps)
    um, uv = sr_noise(numel, sr_tensor_salt(seed, step, tensor_salt))
    mc, ms = quantize_sr(m_new, 0, um)
    vc, rmax, cmax = quantize_rank1_sr(v_new.view(rows, cols), uv)
    return p_new.to(p.dtype).view_as(p), mc, vc, ms, rmax, cmax


def step_quant_sr(p, g, m_codes, v_codes, m_scale, v_scale, *, seed, tensor_salt, beta1, beta2, lr,
                  weight_decay, eps, step):
    """step_quant with stochastic rounding of both moments (CPU tensors)."""
    numel = p.numel()
    sc = derive_scalars(beta1, beta2, lr, weight_decay, step)
    m = dequantize(m_codes, m_scale, numel, 0)
    v = dequantize(v_codes, v_scale, numel, 1)
    p_new, m_new, v_new = adamw_update(p.reshape(-1).float(), g.reshape(-1).float(), m, v, sc, eps)
    um, uv = sr_noise(numel, sr_tensor_salt(seed, step, tensor_salt))
    mc, ms = quantize_sr(m_new, 0, um)
    vc, vs = quantize_sr(v_new, 1, uv)
    return p_new.to(p.dtype).view_as(p), mc, vc, ms, vs


def closed_form_tables():
    """Independent constructions of the four tables (double precision, then fp32):
    second moment k/16 and (2k+1)/32 (quant_opt_base.py:88-102); first moment from
    the dynamic-exponent construction (quant_opt_base.py:55-86): for exponent level
    i = 0..2 the 2**i means of adjacent points of linspace(0.1, 1, 2**i + 1), scaled
    by 10**(i - 2), mirrored, plus 0 and 1.0."""
    pos = []
    for i in range(3):
        n = 2 ** i + 1
        pts = [0.1 + (1.0 - 0.1) * k / (n - 1) for k in range(n)]
        means = [(pts[k] + pts[k + 1]) / 2 for k in range(n - 1)]
        pos += [10.0 ** (i - 2) * x for x in means]
    qm = sorted([-x for x in pos] + [0.0] + pos + [1.0])
    mid_m = [(qm[j] + qm[j + 1]) / 2 for j in range(15)]
    return qm, mid_m, _QMAP_V, _QMID_V
