"""ctypes binding of libq4adamw.so (declarations: include/q4adamw.h).

There is no fallback: if the library is missing, loading raises, and every
optimizer step raises with it.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libq4adamw.so")

FP32, BF16, FP16 = 0, 1, 2
BLOCK = 128


class Q4Tensor(ctypes.Structure):
    """struct q4adamw_tensor"""
    _fields_ = [
        ("p", ctypes.c_void_p),
        ("g", ctypes.c_void_p),
        ("exp_avg", ctypes.c_void_p),
        ("exp_avg_sq", ctypes.c_void_p),
        ("exp_avg_scale", ctypes.c_void_p),
        ("exp_avg_sq_scale", ctypes.c_void_p),
        ("numel", ctypes.c_int64),
    ]


class Q4SmallTensor(ctypes.Structure):
    """struct q4adamw_small_tensor"""
    _fields_ = [
        ("p", ctypes.c_void_p),
        ("g", ctypes.c_void_p),
        ("exp_avg", ctypes.c_void_p),
        ("exp_avg_sq", ctypes.c_void_p),
        ("numel", ctypes.c_int64),
    ]


class Q4Rank1Tensor(ctypes.Structure):
    """struct q4adamw_rank1_tensor"""
    _fields_ = [
        ("p", ctypes.c_void_p),
        ("g", ctypes.c_void_p),
        ("exp_avg", ctypes.c_void_p),
        ("exp_avg_sq", ctypes.c_void_p),
        ("exp_avg_scale", ctypes.c_void_p),
        ("row_max", ctypes.c_void_p),
        ("col_max", ctypes.c_void_p),
        ("row_max_next", ctypes.c_void_p),
        ("col_max_next", ctypes.c_void_p),
        ("rows", ctypes.c_int64),
        ("cols", ctypes.c_int64),
        ("lead_dims", ctypes.c_int32),
        ("reserved", ctypes.c_int32),
        ("lead_shape", ctypes.c_int64 * 3),
        ("lead_max", ctypes.c_void_p * 3),
        ("lead_max_next", ctypes.c_void_p * 3),
    ]


class Q4GradOptions(ctypes.Structure):
    """struct q4adamw_grad_options"""
    _fields_ = [
        ("grad_scale", ctypes.c_float),
        ("zero_grad", ctypes.c_int),
        ("grad_scale_dev", ctypes.c_void_p),
        ("skip_if_nonzero", ctypes.c_void_p),
        ("step_consts", ctypes.c_void_p),
        ("update_form", ctypes.c_int),
        ("reserved", ctypes.c_int),
    ]


class Q4Grad(ctypes.Structure):
    """struct q4adamw_grad"""
    _fields_ = [
        ("g", ctypes.c_void_p),
        ("numel", ctypes.c_int64),
    ]


NORM_WORKSPACE_BYTES = 16384
STEP_CONSTS_BYTES = 64
# q4adamw_grad_options.update_form (include/q4adamw.h)
UPDATE_AUTO, UPDATE_EXACT, UPDATE_FOLDED = 0, 1, 2
UPDATE_FORMS = {"auto": UPDATE_AUTO, "exact": UPDATE_EXACT, "folded": UPDATE_FOLDED}

EXPORTS = (
    "q4adamw_fused_4bit",
    "q4adamw_fused_4bit_multi",
    "q4adamw_fused_4bit_multi_ex",
    "q4adamw_fused_4bit_multi_sr",
    "q4adamw_sr_tensor_salt",
    "q4adamw_fused_4bit_rank1_multi",
    "q4adamw_fused_4bit_rank1_multi_sr",
    "q4adamw_fused_single_tensor",
    "q4adamw_fused_single_tensor_multi",
    "q4adamw_fused_single_tensor_multi_ex",
    "q4adamw_grad_norm",
    "q4adamw_grad_norm_static",
    "q4adamw_bias_table",
    "q4adamw_device_step",
    "q4adamw_quantize",
    "q4adamw_dequantize",
    "q4adamw_quantize_rank1",
    "q4adamw_quantize_rank1_scaled",
    "q4adamw_dequantize_rank1",
    "q4adamw_derive_scalars",
    "q4adamw_tables",
    "q4adamw_mtable_entry",
    "q4adamw_mtable_half_bucket",
    "q4adamw_sr_bucket_entry",
    "q4adamw_sr_affine_entry",
    "q4adamw_rounding_selfcheck",
    "q4adamw_grid_plan",
    "q4adamw_rank1_form",
    "q4adamw_set_grid_limit",
    "q4adamw_release",
    "q4adamw_last_error",
    "q4adamw_version",
)

_lib = None


def load():
    """Returns the loaded library; raises RuntimeError when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m quantfour_adamw_cuda_amd.build` "
            "(needs hipcc); the 4-bit AdamW step has no other implementation")
    L = ctypes.CDLL(LIB_PATH)
    f, i, i64, vp = ctypes.c_float, ctypes.c_int, ctypes.c_int64, ctypes.c_void_p
    hyper = [f, f, f, f, f, f]  # beta1, beta2, lr, weight_decay, eps, step
    L.q4adamw_fused_4bit.argtypes = [vp, vp, vp, vp, vp, vp, i64, i, i] + hyper + [vp]
    L.q4adamw_fused_4bit.restype = i
    L.q4adamw_fused_4bit_multi.argtypes = [ctypes.POINTER(Q4Tensor), i, i, i] + hyper + [vp]
    L.q4adamw_fused_4bit_multi.restype = i
    L.q4adamw_fused_single_tensor.argtypes = [vp, vp, vp, vp, i64, i, i] + hyper + [vp]
    L.q4adamw_fused_single_tensor.restype = i
    L.q4adamw_fused_single_tensor_multi.argtypes = [ctypes.POINTER(Q4SmallTensor), i, i, i] + hyper + [vp]
    L.q4adamw_fused_single_tensor_multi.restype = i
    opt = ctypes.POINTER(Q4GradOptions)
    L.q4adamw_fused_4bit_multi_ex.argtypes = [ctypes.POINTER(Q4Tensor), i, i, i] + hyper + [opt, vp]
    L.q4adamw_fused_4bit_multi_ex.restype = i
    L.q4adamw_fused_single_tensor_multi_ex.argtypes = [ctypes.POINTER(Q4SmallTensor), i, i, i] + hyper + [opt, vp]
    L.q4adamw_fused_single_tensor_multi_ex.restype = i
    L.q4adamw_fused_4bit_multi_sr.argtypes = ([ctypes.POINTER(Q4Tensor), i, ctypes.POINTER(ctypes.c_uint32),
                                               ctypes.c_uint64, i, i] + hyper + [opt, vp])
    L.q4adamw_fused_4bit_multi_sr.restype = i
    L.q4adamw_sr_tensor_salt.argtypes = [ctypes.c_uint64, f, ctypes.c_uint32]
    L.q4adamw_sr_tensor_salt.restype = ctypes.c_uint32
    L.q4adamw_fused_4bit_rank1_multi.argtypes = [ctypes.POINTER(Q4Rank1Tensor), i, i, i] + hyper + [opt, vp]
    L.q4adamw_fused_4bit_rank1_multi.restype = i
    L.q4adamw_fused_4bit_rank1_multi_sr.argtypes = ([ctypes.POINTER(Q4Rank1Tensor), i,
                                                     ctypes.POINTER(ctypes.c_uint32), ctypes.c_uint64, i, i]
                                                    + hyper + [opt, vp])
    L.q4adamw_fused_4bit_rank1_multi_sr.restype = i
    L.q4adamw_grad_norm.argtypes = [ctypes.POINTER(Q4Grad), i, i, f, vp, f, vp, ctypes.c_size_t, vp, vp]
    L.q4adamw_grad_norm.restype = i
    L.q4adamw_grad_norm_static.argtypes = [ctypes.POINTER(Q4Grad), i, i, f, vp, f, vp, vp]
    L.q4adamw_grad_norm_static.restype = i
    L.q4adamw_bias_table.argtypes = [f, f, i64, i64, vp]
    L.q4adamw_bias_table.restype = i
    L.q4adamw_device_step.argtypes = [vp, vp, i64, i64, vp, f, f, f, f, f, vp, vp, vp]
    L.q4adamw_device_step.restype = i
    L.q4adamw_quantize.argtypes = [vp, i64, i, vp, vp, vp]
    L.q4adamw_quantize.restype = i
    L.q4adamw_dequantize.argtypes = [vp, vp, i64, i, vp, vp]
    L.q4adamw_dequantize.restype = i
    L.q4adamw_quantize_rank1.argtypes = [vp, i64, i64, vp, vp, vp, vp]
    L.q4adamw_quantize_rank1.restype = i
    L.q4adamw_quantize_rank1_scaled.argtypes = [vp, i64, i64, vp, vp, vp, vp]
    L.q4adamw_quantize_rank1_scaled.restype = i
    L.q4adamw_dequantize_rank1.argtypes = [vp, vp, vp, i64, i64, vp, vp]
    L.q4adamw_dequantize_rank1.restype = i
    L.q4adamw_derive_scalars.argtypes = [f, f, f, f, f, ctypes.POINTER(f)]
    L.q4adamw_derive_scalars.restype = None
    L.q4adamw_tables.argtypes = [i, ctypes.POINTER(f), ctypes.POINTER(f)]
    L.q4adamw_tables.restype = None
    L.q4adamw_mtable_entry.argtypes = [ctypes.c_uint32, ctypes.POINTER(ctypes.c_uint32)]
    L.q4adamw_mtable_entry.restype = i
    L.q4adamw_mtable_half_bucket.argtypes = [ctypes.c_uint32]
    L.q4adamw_mtable_half_bucket.restype = i
    L.q4adamw_sr_bucket_entry.argtypes = [ctypes.c_uint32, ctypes.POINTER(ctypes.c_uint32)]
    L.q4adamw_sr_bucket_entry.restype = i
    L.q4adamw_sr_affine_entry.argtypes = [ctypes.c_uint32, ctypes.POINTER(ctypes.c_float)]
    L.q4adamw_sr_affine_entry.restype = i
    L.q4adamw_rounding_selfcheck.argtypes = [vp, vp]
    L.q4adamw_grid_plan.argtypes = [ctypes.c_uint64, i, ctypes.POINTER(ctypes.c_uint64), ctypes.POINTER(ctypes.c_uint64), i]
    L.q4adamw_grid_plan.restype = i
    L.q4adamw_rank1_form.argtypes = [i64, i64, i]
    L.q4adamw_rank1_form.restype = i
    L.q4adamw_set_grid_limit.argtypes = [ctypes.c_uint64]
    L.q4adamw_set_grid_limit.restype = None
    L.q4adamw_rounding_selfcheck.restype = i
    L.q4adamw_release.argtypes = []
    L.q4adamw_release.restype = i
    L.q4adamw_last_error.argtypes = []
    L.q4adamw_last_error.restype = ctypes.c_char_p
    L.q4adamw_version.argtypes = []
    L.q4adamw_version.restype = i
    _lib = L
    return L


def check(status, what):
    """Turns a non-zero status into the RuntimeError the reference's bindings raise
    from AT_CUDA_CHECK / AT_ASSERTM (optim/cuda_adamw_kernels.cu:140, :163, :468)."""
    if status != 0:
        msg = load().q4adamw_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{what} failed with status {status}: {msg}")
