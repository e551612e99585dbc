"""TEST INFRASTRUCTURE -- ctypes binding of the scalar C oracle (q4_oracle.c).

A checker, not a product path: only tests/, the smoke check and the cpu_baseline
leg of bench.py import this module.  See the header of q4_oracle.c for what each
function restates (reference file:line) and for its pinning status.

All tensors are numpy arrays (or anything exposing the buffer protocol through
``numpy.asarray``) that are updated IN PLACE, like the reference's kernels update
their torch tensors in place (optim/cuda_fused_interface.cc:19-39).
bf16 data is passed as uint16 bit patterns, fp16 data as numpy float16.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libq4oracle.so")

BLOCK = 128
FP32, BF16, FP16 = 0, 1, 2


def build(force=False):
    """Compile q4_oracle.c with gcc (seconds)."""
    if force or not os.path.exists(_SO) or (
        os.path.getmtime(_SO) < os.path.getmtime(os.path.join(_HERE, "q4_oracle.c"))
    ):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libq4oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_SO)
        f, i64, vp, ci = ctypes.c_float, ctypes.c_int64, ctypes.c_void_p, ctypes.c_int
        L.q4o_tables.argtypes = [ci, vp, vp]
        L.q4o_quantize_search.argtypes = [ci, f]
        L.q4o_quantize_search.restype = ci
        L.q4o_quantize_count.argtypes = [ci, f]
        L.q4o_quantize_count.restype = ci
        L.q4o_derive_scalars.argtypes = [f, f, f, f, f, vp]
        L.q4o_step_quant.argtypes = [vp, vp, vp, vp, vp, vp, i64, ci, ci, f, f, f, f, f, f]
        L.q4o_step_unquant.argtypes = [vp, vp, vp, vp, i64, ci, ci, f, f, f, f, f, f]
        L.q4o_dequant.argtypes = [vp, vp, i64, ci, vp]
        L.q4o_quant.argtypes = [vp, i64, ci, vp, vp]
        u32, u64 = ctypes.c_uint32, ctypes.c_uint64
        L.q4o_step_quant_variants.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, ci, i64, ci, ci, f, f, f, f, f, f,
                                              ci, u64, u32, vp]
        L.q4o_sr_tensor_salt.argtypes = [u64, u32, u32]
        L.q4o_sr_tensor_salt.restype = u32
        L.q4o_sr_noise.argtypes = [i64, u32, vp, vp]
        L.q4o_quantize_sr.argtypes = [ci, f, f]
        L.q4o_quantize_sr.restype = ci
        L.q4o_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.q4o_f16_to_f32.restype = f
        L.q4o_f32_to_f16.argtypes = [f]
        L.q4o_f32_to_f16.restype = ctypes.c_uint16
        _lib = L
    return _lib


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _dtype_tag(a):
    if a.dtype == np.float32:
        return FP32
    if a.dtype == np.float16:
        return FP16
    if a.dtype == np.uint16:
        return BF16
    raise TypeError(f"expected float32, float16 or uint16 (bf16 bits), got {a.dtype}")


def tables(which):
    """(qmap[16], qmid[15]) as float32 arrays; which 0 = first moment, 1 = second."""
    qmap = np.empty(16, np.float32)
    qmid = np.empty(15, np.float32)
    lib().q4o_tables(which, _ptr(qmap), _ptr(qmid))
    return qmap, qmid


def quantize_search(which, x):
    return lib().q4o_quantize_search(which, float(np.float32(x)))


def quantize_count(which, x):
    return lib().q4o_quantize_count(which, float(np.float32(x)))


def exhaustive_search_vs_count(which):
    """(mismatching bit patterns, lowest mismatching pattern, steps of the staircase) over all
    2^32 fp32 bit patterns; takes about a quarter of a minute on 8 cores."""
    L = lib()
    L.q4o_exhaustive_search_vs_count.restype = ctypes.c_int64
    first, steps = ctypes.c_uint32(0), ctypes.c_int64(0)
    bad = L.q4o_exhaustive_search_vs_count(int(which), ctypes.byref(first), ctypes.byref(steps))
    return int(bad), int(first.value), int(steps.value)


def derive_scalars(beta1, beta2, lr, weight_decay, step):
    """fp32 {correction1, correction2_sqrt, step_size, weight_decay_update,
    resid_beta1, resid_beta2} exactly as the reference launcher derives them."""
    out = np.empty(6, np.float32)
    lib().q4o_derive_scalars(beta1, beta2, lr, weight_decay, float(step), _ptr(out))
    return out


def state_sizes(numel):
    """(code bytes per state, scales per state) for a tensor of numel elements."""
    return (numel + 1) // 2, (numel + BLOCK - 1) // BLOCK


def step_quant(p, g, m_codes, v_codes, m_scale, v_scale, *, beta1, beta2, lr,
               weight_decay, eps, step):
    n = p.size
    nbytes, nblk = state_sizes(n)
    assert g.size == n and m_codes.size == nbytes and v_codes.size == nbytes
    assert m_scale.size == nblk and v_scale.size == nblk
    assert m_codes.dtype == np.uint8 and v_codes.dtype == np.uint8
    assert m_scale.dtype == np.float32 and v_scale.dtype == np.float32
    for a in (p, g, m_codes, v_codes, m_scale, v_scale):
        assert a.flags.c_contiguous
    lib().q4o_step_quant(_ptr(p), _ptr(g), _ptr(m_codes), _ptr(v_codes), _ptr(m_scale),
                         _ptr(v_scale), n, _dtype_tag(p), _dtype_tag(g), beta1, beta2, lr,
                         weight_decay, eps, float(step))


def step_quant_variants(p, g, m_codes, v_codes, m_scale, v_scale=None, row_max=None, col_max=None, *, beta1,
                        beta2, lr, weight_decay, eps, step, seed=None, tensor_salt=0, max_dims=None):
    """The fused step with its options, in place.  row_max / col_max given (p a [rows, cols]
    matrix), or max_dims = one float32 array per dimension of p: rank-1 scaled second moment;
    else v_scale = per-128 block scales.  seed given = stochastic rounding with the noise of
    (seed, step, tensor_salt)."""
    if row_max is not None:
        max_dims = [row_max, col_max]
    rank1 = max_dims is not None
    n = p.size
    nbytes, nblk = state_sizes(n)
    assert g.size == n and m_codes.size == nbytes and v_codes.size == nbytes and m_scale.size == nblk
    assert m_codes.dtype == np.uint8 and v_codes.dtype == np.uint8 and m_scale.dtype == np.float32
    none = ctypes.c_void_p(0)
    if rank1:
        assert v_scale is None and len(max_dims) == p.ndim >= 2
        assert all(s.size == d and s.dtype == np.float32 and s.flags.c_contiguous for s, d in zip(max_dims, p.shape))
        shape = (ctypes.c_int64 * p.ndim)(*p.shape)
        stats = (ctypes.c_void_p * p.ndim)(*[s.ctypes.data for s in max_dims])
    else:
        assert v_scale.size == nblk and v_scale.dtype == np.float32 and v_scale.flags.c_contiguous
        shape, stats = none, none
    for a in (p, g, m_codes, v_codes, m_scale):
        assert a.flags.c_contiguous
    scratch = np.empty(2 * n, np.float32)
    lib().q4o_step_quant_variants(_ptr(p), _ptr(g), _ptr(m_codes), _ptr(v_codes), _ptr(m_scale),
                                  none if rank1 else _ptr(v_scale), stats, shape, p.ndim if rank1 else 0, n,
                                  _dtype_tag(p), _dtype_tag(g), beta1, beta2, lr, weight_decay, eps, float(step),
                                  int(seed is not None), int(seed or 0) & (2 ** 64 - 1),
                                  int(tensor_salt) & 0xFFFFFFFF, _ptr(scratch))


def sr_tensor_salt(seed, step, tensor_salt):
    return int(lib().q4o_sr_tensor_salt(int(seed) & (2 ** 64 - 1), int(step) & 0xFFFFFFFF,
                                        int(tensor_salt) & 0xFFFFFFFF))


def sr_noise(e, salt):
    """(first-moment noise, second-moment noise) of element e"""
    um, uv = ctypes.c_float(), ctypes.c_float()
    lib().q4o_sr_noise(int(e), int(salt) & 0xFFFFFFFF, ctypes.byref(um), ctypes.byref(uv))
    return um.value, uv.value


def quantize_sr(which, q, u):
    return int(lib().q4o_quantize_sr(which, q, u))


def step_unquant(p, g, m, v, *, beta1, beta2, lr, weight_decay, eps, step):
    n = p.size
    assert g.size == n and m.size == n and v.size == n
    assert m.dtype == np.float32 and v.dtype == np.float32
    for a in (p, g, m, v):
        assert a.flags.c_contiguous
    lib().q4o_step_unquant(_ptr(p), _ptr(g), _ptr(m), _ptr(v), n, _dtype_tag(p),
                           _dtype_tag(g), beta1, beta2, lr, weight_decay, eps, float(step))


def dequant(codes, scale, numel, which):
    out = np.empty(numel, np.float32)
    lib().q4o_dequant(_ptr(codes), _ptr(scale), numel, which, _ptr(out))
    return out


def quant(x, which):
    x = np.ascontiguousarray(x, np.float32).ravel()
    nbytes, nblk = state_sizes(x.size)
    codes = np.zeros(nbytes, np.uint8)
    scale = np.zeros(nblk, np.float32)
    lib().q4o_quant(_ptr(x), x.size, which, _ptr(codes), _ptr(scale))
    return codes, scale


# ---------------------------------------------------------------------------
# gradient-side operations folded into the step
#
# The reference has no code for these: its callers zero, unscale and clip the
# gradients around step() with torch's own routines (caller pattern:
# tests/driver.py:53-59).  What is restated here is the published arithmetic of
# those routines: GradScaler.unscale_ multiplies every gradient by a reciprocal
# scale in fp32; torch.nn.utils.clip_grad_norm_ multiplies by
# min(1, max_norm / (total_norm + 1e-6)).  Pinned against torch's routines on the
# CPU (tests/test_oracle_pins.py); parity with the reference itself: UNPINNED, it
# has no counterpart.
# ---------------------------------------------------------------------------
def as_f32(g):
    """fp32 values of a gradient given as float32, float16 or as bf16 bit patterns (uint16)."""
    g = np.asarray(g)
    if g.dtype == np.uint16:
        return (g.astype(np.uint32) << 16).view(np.float32)
    return g.astype(np.float32, copy=False)


def scale_grad(g, s):
    """The gradient a step with multiplier s works on: one rounded fp32 product per
    element.  Feed the result to step_quant / step_unquant as a float32 gradient."""
    return as_f32(g) * np.float32(s)


def grad_norm(gs, s=1.0, max_norm=0.0):
    """(norm of the gradients times s, clip coefficient, s * coefficient), fp32 each:
    squares summed in fp64, the rest in fp32 in torch's order."""
    total = 0.0
    for g in gs:
        x = as_f32(g).astype(np.float64)
        total += float(np.dot(x, x))
    s = np.float32(s)
    norm = np.float32(np.abs(s) * np.float32(np.sqrt(total)))
    coef = np.float32(1.0)
    if max_norm > 0.0:
        with np.errstate(over="ignore", invalid="ignore"):
            coef = np.float32(max_norm) / (norm + np.float32(1e-6))
        coef = np.float32(1.0) if coef > 1.0 else np.float32(coef)
    return norm, coef, np.float32(s * coef)
