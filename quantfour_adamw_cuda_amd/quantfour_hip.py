"""Tensor-level entry points: the stand-in for the reference's compiled module
`quantfour_cuda` (optim/cuda_fused_interface.cc:66-69, imported at
optim/fused_quantfour.py:10).

`fused_4bit` and `fused_single_tensor` keep the reference's positional signature
(param, grad, moments, scales, beta1, beta2, lr, weight_decay, eps, step); the
`*_multi` forms take lists of tensors and replace the reference's per-parameter
Python loop by one launch.  All tensors are updated in place and the call is
asynchronous on torch's current stream of the tensors' device.
"""
import torch

from . import _lib

_DTYPE_TAG = {torch.float32: _lib.FP32, torch.bfloat16: _lib.BF16}


def state_sizes(numel):
    """(bytes of packed codes per moment, fp32 scales per moment)."""
    return (numel + 1) // 2, (numel + _lib.BLOCK - 1) // _lib.BLOCK


def _tag(t, what):
    try:
        return _DTYPE_TAG[t.dtype]
    except KeyError:
        raise TypeError(f"{what} must be float32 or bfloat16, got {t.dtype}") from None


def _check_common(p, g):
    # optim/fused_quantfour.py:255-261
    assert p.is_cuda, "param must be on cuda"
    assert p.is_contiguous(), "param must be contiguous"
    assert g.is_cuda and g.device == p.device, "grad must be on the param's device"
    assert g.is_contiguous(), "grad must be contiguous"
    assert g.numel() == p.numel(), f"grad numel {g.numel()} != param numel {p.numel()}"


def check_quantized(p, g, exp, sq, exp_scale, sq_scale):
    _check_common(p, g)
    nbytes, nblk = state_sizes(p.numel())
    assert exp.dtype == torch.uint8 and sq.dtype == torch.uint8, "moments must be packed uint8"
    assert exp.numel() == nbytes, f"exp_avg numel {exp.numel()} != packed size {nbytes}"
    assert sq.numel() == nbytes, f"exp_avg_sq numel {sq.numel()} != packed size {nbytes}"
    assert exp_scale.dtype == torch.float32 and sq_scale.dtype == torch.float32, "scales must be float32"
    assert exp_scale.numel() == nblk and sq_scale.numel() == nblk, f"scales must hold {nblk} blocks"
    for t in (exp, sq, exp_scale, sq_scale):
        assert t.device == p.device and t.is_contiguous(), "state must be contiguous on the param's device"


def check_unquantized(p, g, exp_avg, exp_avg_sq):
    _check_common(p, g)
    for t in (exp_avg, exp_avg_sq):
        assert t.dtype == torch.float32, "non-quantized moments must be float32"
        assert t.numel() == p.numel(), f"moment numel {t.numel()} != param numel {p.numel()}"
        assert t.device == p.device and t.is_contiguous(), "state must be contiguous on the param's device"


def _stream(device):
    return torch.cuda.current_stream(device).cuda_stream


def fused_4bit(p, g, exp, sq, exp_scale, sq_scale, beta1, beta2, lr, weight_decay, eps, step):
    """optim/cuda_fused_interface.cc:19-39."""
    L = _lib.load()
    check_quantized(p, g, exp, sq, exp_scale, sq_scale)
    with torch.cuda.device(p.device):
        rc = L.q4adamw_fused_4bit(p.data_ptr(), g.data_ptr(), exp.data_ptr(), sq.data_ptr(),
                                  exp_scale.data_ptr(), sq_scale.data_ptr(), p.numel(),
                                  _tag(p, "param"), _tag(g, "grad"), beta1, beta2, lr,
                                  weight_decay, eps, float(step), _stream(p.device))
    _lib.check(rc, "fused_4bit")


def fused_single_tensor(p, g, exp_avg, exp_avg_sq, beta1, beta2, lr, weight_decay, eps, step):
    """optim/cuda_fused_interface.cc:49-64."""
    L = _lib.load()
    check_unquantized(p, g, exp_avg, exp_avg_sq)
    with torch.cuda.device(p.device):
        rc = L.q4adamw_fused_single_tensor(p.data_ptr(), g.data_ptr(), exp_avg.data_ptr(),
                                           exp_avg_sq.data_ptr(), p.numel(), _tag(p, "param"),
                                           _tag(g, "grad"), beta1, beta2, lr, weight_decay, eps,
                                           float(step), _stream(p.device))
    _lib.check(rc, "fused_single_tensor")


def make_table(ps, gs, exps, sqs, exp_scales, sq_scales):
    """ctypes descriptor array for fused_4bit_multi_table (all tensors validated)."""
    n = len(ps)
    arr = (_lib.Q4Tensor * n)()
    for i in range(n):
        check_quantized(ps[i], gs[i], exps[i], sqs[i], exp_scales[i], sq_scales[i])
        a = arr[i]
        a.p, a.g = ps[i].data_ptr(), gs[i].data_ptr()
        a.exp_avg, a.exp_avg_sq = exps[i].data_ptr(), sqs[i].data_ptr()
        a.exp_avg_scale, a.exp_avg_sq_scale = exp_scales[i].data_ptr(), sq_scales[i].data_ptr()
        a.numel = ps[i].numel()
    return arr


def make_small_table(ps, gs, exp_avgs, exp_avg_sqs):
    n = len(ps)
    arr = (_lib.Q4SmallTensor * n)()
    for i in range(n):
        check_unquantized(ps[i], gs[i], exp_avgs[i], exp_avg_sqs[i])
        a = arr[i]
        a.p, a.g = ps[i].data_ptr(), gs[i].data_ptr()
        a.exp_avg, a.exp_avg_sq = exp_avgs[i].data_ptr(), exp_avg_sqs[i].data_ptr()
        a.numel = ps[i].numel()
    return arr


def launch_table(arr, device, p_tag, g_tag, beta1, beta2, lr, weight_decay, eps, step):
    L = _lib.load()
    with torch.cuda.device(device):
        rc = L.q4adamw_fused_4bit_multi(arr, len(arr), p_tag, g_tag, beta1, beta2, lr,
                                        weight_decay, eps, float(step), _stream(device))
    _lib.check(rc, "fused_4bit_multi")


def launch_small_table(arr, device, p_tag, g_tag, beta1, beta2, lr, weight_decay, eps, step):
    L = _lib.load()
    with torch.cuda.device(device):
        rc = L.q4adamw_fused_single_tensor_multi(arr, len(arr), p_tag, g_tag, beta1, beta2, lr,
                                                 weight_decay, eps, float(step), _stream(device))
    _lib.check(rc, "fused_single_tensor_multi")


def fused_4bit_multi(ps, gs, exps, sqs, exp_scales, sq_scales, beta1, beta2, lr, weight_decay,
                     eps, step):
    """One launch over many quantized tensors that share device, dtypes and step."""
    if not ps:
        return
    arr = make_table(ps, gs, exps, sqs, exp_scales, sq_scales)
    p_tag, g_tag = _tag(ps[0], "param"), _tag(gs[0], "grad")
    for p, g in zip(ps, gs):
        assert p.device == ps[0].device and _tag(p, "param") == p_tag and _tag(g, "grad") == g_tag, \
            "tensors of one launch must share device and dtypes"
    launch_table(arr, ps[0].device, p_tag, g_tag, beta1, beta2, lr, weight_decay, eps, step)


def fused_single_tensor_multi(ps, gs, exp_avgs, exp_avg_sqs, beta1, beta2, lr, weight_decay,
                              eps, step):
    """One launch over many non-quantized tensors that share device, dtypes and step."""
    if not ps:
        return
    arr = make_small_table(ps, gs, exp_avgs, exp_avg_sqs)
    p_tag, g_tag = _tag(ps[0], "param"), _tag(gs[0], "grad")
    for p, g in zip(ps, gs):
        assert p.device == ps[0].device and _tag(p, "param") == p_tag and _tag(g, "grad") == g_tag, \
            "tensors of one launch must share device and dtypes"
    launch_small_table(arr, ps[0].device, p_tag, g_tag, beta1, beta2, lr, weight_decay, eps, step)


def quantize_state(x, which):
    """fp32 moment (any shape, on a GPU) -> (packed uint8 codes, fp32 block scales).
    which: 0 first moment, 1 second moment.  Device form of momentum_quant /
    variance_quant with per-block scaling (optim/adamw_fourbit_triton.py:556-630)."""
    L = _lib.load()
    assert x.is_cuda, "state must be on cuda"
    x = x.detach().to(torch.float32).contiguous().reshape(-1)
    nbytes, nblk = state_sizes(x.numel())
    codes = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    scales = torch.empty(nblk, dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        rc = L.q4adamw_quantize(x.data_ptr(), x.numel(), int(which), codes.data_ptr(),
                                scales.data_ptr(), _stream(x.device))
    _lib.check(rc, "quantize")
    return codes, scales


def dequantize_state(codes, scales, numel, which):
    """(packed codes, block scales) -> flat fp32 moment of numel elements
    (optim/cuda_adamw_kernels.cu:329-343)."""
    L = _lib.load()
    assert codes.is_cuda and scales.device == codes.device, "state must be on cuda"
    nbytes, nblk = state_sizes(numel)
    assert codes.dtype == torch.uint8 and codes.numel() == nbytes and codes.is_contiguous()
    assert scales.dtype == torch.float32 and scales.numel() == nblk and scales.is_contiguous()
    out = torch.empty(numel, dtype=torch.float32, device=codes.device)
    with torch.cuda.device(codes.device):
        rc = L.q4adamw_dequantize(codes.data_ptr(), scales.data_ptr(), numel, int(which),
                                  out.data_ptr(), _stream(codes.device))
    _lib.check(rc, "dequantize")
    return out
