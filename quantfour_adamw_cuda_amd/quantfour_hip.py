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

_DTYPE_TAG = {torch.float32: _lib.FP32, torch.bfloat16: _lib.BF16, torch.float16: _lib.FP16}


def state_sizes(numel):
    """(bytes of packed codes per moment, fp32 scales per moment)."""
    return (numel + 1) // 2, (numel + _lib.BLOCK - 1) // _lib.BLOCK


def _tag(t, what):
    try:
        return _DTYPE_TAG[t.dtype]
    except KeyError:
        raise TypeError(f"{what} must be float32, bfloat16 or float16, got {t.dtype}") from None


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


class _OnDevice:
    """`with _on(device):` -- torch.cuda.device(device) when another device is current, else
    nothing (the step's launches run in a loop where the context switch would cost as much
    as the launch)."""
    __slots__ = ("ctx",)

    def __init__(self, device):
        self.ctx = None if torch.cuda.current_device() == device.index else torch.cuda.device(device)

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()

    def __exit__(self, *exc):
        if self.ctx is not None:
            return self.ctx.__exit__(*exc)
        return False


_on = _OnDevice


def fused_4bit(p, g, exp, sq, exp_scale, sq_scale, beta1, beta2, lr, weight_decay, eps, step,
               update_form="auto"):
    """optim/cuda_fused_interface.cc:19-39.  update_form ("auto", "exact", "folded"): how the
    parameter is computed, see grad_options; anything but "auto" goes through the multi-tensor
    entry point, which takes options."""
    if update_form != "auto":
        return fused_4bit_multi([p], [g], [exp], [sq], [exp_scale], [sq_scale], beta1, beta2, lr,
                                weight_decay, eps, step, update_form=update_form)
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


def _device_scalar(t, device, what):
    assert t.is_cuda and t.device == device, f"{what} must be on the tensors' device"
    assert t.dtype == torch.float32 and t.numel() == 1, f"{what} must hold one float32"
    return t.data_ptr()


def grad_options(device, grad_scale=1.0, grad_scale_dev=None, found_inf=None, zero_grad=False,
                 step_consts=None, update_form="auto"):
    """struct q4adamw_grad_options, or None when the arguments change nothing.  The device
    scalars are referenced, not copied: keep the tensors alive until the step has run.
    step_consts: the buffer device_step() filled, for a step whose number lives on the device.
    update_form: "exact" = the parameter update of optim/cuda_adamw_kernels.cu:334,351 with every
    operation rounded as IEEE 754 rounds it (parameters bit-identical to that expression),
    "folded" = the short form with hardware square root and reciprocal (a tolerance), "auto" =
    exact where it is nearly free (fp32 parameters, block scales, nearest rounding)."""
    form = _lib.UPDATE_FORMS.get(update_form)
    if form is None:
        raise ValueError(f"Invalid update_form: {update_form=}")
    if (grad_scale == 1.0 and grad_scale_dev is None and found_inf is None and not zero_grad
            and step_consts is None and form == _lib.UPDATE_AUTO):
        return None
    o = _lib.Q4GradOptions()
    o.update_form = form
    o.grad_scale = float(grad_scale)
    o.zero_grad = 1 if zero_grad else 0
    o.grad_scale_dev = None if grad_scale_dev is None else _device_scalar(grad_scale_dev, device, "grad_scale_dev")
    o.skip_if_nonzero = None if found_inf is None else _device_scalar(found_inf, device, "found_inf")
    if step_consts is not None:
        assert step_consts.is_cuda and step_consts.device == device and step_consts.is_contiguous()
        assert step_consts.numel() * step_consts.element_size() >= _lib.STEP_CONSTS_BYTES, "step_consts too small"
        o.step_consts = step_consts.data_ptr()
    return o


def make_bias_table(beta1, beta2, device, max_steps=1 << 22):
    """Device table of (1 - beta1^t, sqrt(1 - beta2^t)) for t = 1 .. T, two floats per step,
    computed as the step's launcher computes them; T is the first power of two (from 1024)
    at which both have become exactly 1, so that later steps may take the last entry."""
    import ctypes
    L = _lib.load()
    steps = 1024
    while True:
        last = (ctypes.c_float * 2)()
        _lib.check(L.q4adamw_bias_table(beta1, beta2, steps, 1, last), "bias_table")
        if last[0] == 1.0 and last[1] == 1.0:
            break
        if steps >= max_steps:
            raise ValueError(f"bias corrections of betas ({beta1}, {beta2}) have not reached 1 after {steps} steps")
        steps *= 2
    host = torch.empty(steps, 2, dtype=torch.float32)
    _lib.check(L.q4adamw_bias_table(beta1, beta2, 1, steps, host.data_ptr()), "bias_table")
    return host.to(device)


def new_step_consts(device):
    """Device buffer for device_step() to fill and grad_options(step_consts=...) to pass on."""
    return torch.zeros(_lib.STEP_CONSTS_BYTES // 4, dtype=torch.float32, device=device)


def device_step(step, table, consts, beta1, beta2, lr, weight_decay, eps, lr_dev=None, found_inf=None):
    """Adds 1 to the device step counter `step` (one float32) unless found_inf holds a
    non-zero value, and leaves the new step's derived scalars in `consts`; lr comes from the
    device scalar lr_dev if given.  Asynchronous on the current stream; captures into a graph."""
    L = _lib.load()
    device = step.device
    assert step.is_cuda and step.dtype == torch.float32 and step.numel() == 1, "step must be one device float32"
    assert table.device == device and table.dtype == torch.float32 and table.dim() == 2 and table.shape[1] == 2 \
        and table.is_contiguous(), "table must come from make_bias_table"
    assert consts.device == device and consts.numel() * consts.element_size() >= _lib.STEP_CONSTS_BYTES
    lr_ptr = None if lr_dev is None else _device_scalar(lr_dev, device, "lr_dev")
    skip = None if found_inf is None else _device_scalar(found_inf, device, "found_inf")
    with torch.cuda.device(device):
        rc = L.q4adamw_device_step(step.data_ptr(), table.data_ptr(), 1, table.shape[0], lr_ptr, beta1, beta2,
                                   float(lr), weight_decay, eps, skip, consts.data_ptr(), _stream(device))
    _lib.check(rc, "device_step")


def launch_table(arr, device, p_tag, g_tag, beta1, beta2, lr, weight_decay, eps, step, options=None):
    L = _lib.load()
    with _on(device):
        rc = L.q4adamw_fused_4bit_multi_ex(arr, len(arr), p_tag, g_tag, beta1, beta2, lr,
                                           weight_decay, eps, float(step), options, _stream(device))
    _lib.check(rc, "fused_4bit_multi")


def launch_small_table(arr, device, p_tag, g_tag, beta1, beta2, lr, weight_decay, eps, step,
                       options=None):
    L = _lib.load()
    with _on(device):
        rc = L.q4adamw_fused_single_tensor_multi_ex(arr, len(arr), p_tag, g_tag, beta1, beta2, lr,
                                                    weight_decay, eps, float(step), options,
                                                    _stream(device))
    _lib.check(rc, "fused_single_tensor_multi")


def fused_4bit_multi(ps, gs, exps, sqs, exp_scales, sq_scales, beta1, beta2, lr, weight_decay,
                     eps, step, grad_scale=1.0, grad_scale_dev=None, found_inf=None, zero_grad=False,
                     step_consts=None, update_form="auto"):
    """One launch over many quantized tensors that share device, dtypes and step.  The
    gradients enter the step multiplied by grad_scale * grad_scale_dev (a device float32
    scalar); found_inf (a device float32 scalar) makes the call leave parameters and state
    alone when it holds a non-zero value; zero_grad overwrites the gradients with zeros once
    they are read, also in a call that found_inf cancels.  step_consts (filled by device_step)
    replaces the scalars derived from lr, weight_decay, eps and step."""
    if not ps:
        return
    arr = make_table(ps, gs, exps, sqs, exp_scales, sq_scales)
    p_tag, g_tag = _tag(ps[0], "param"), _tag(gs[0], "grad")
    for p, g in zip(ps, gs):
        assert p.device == ps[0].device and _tag(p, "param") == p_tag and _tag(g, "grad") == g_tag, \
            "tensors of one launch must share device and dtypes"
    options = grad_options(ps[0].device, grad_scale, grad_scale_dev, found_inf, zero_grad, step_consts,
                           update_form)
    launch_table(arr, ps[0].device, p_tag, g_tag, beta1, beta2, lr, weight_decay, eps, step, options)


def fused_single_tensor_multi(ps, gs, exp_avgs, exp_avg_sqs, beta1, beta2, lr, weight_decay,
                              eps, step, grad_scale=1.0, grad_scale_dev=None, found_inf=None,
                              zero_grad=False, step_consts=None):
    """One launch over many non-quantized tensors that share device, dtypes and step; gradient
    options as for fused_4bit_multi."""
    if not ps:
        return
    arr = make_small_table(ps, gs, exp_avgs, exp_avg_sqs)
    p_tag, g_tag = _tag(ps[0], "param"), _tag(gs[0], "grad")
    for p, g in zip(ps, gs):
        assert p.device == ps[0].device and _tag(p, "param") == p_tag and _tag(g, "grad") == g_tag, \
            "tensors of one launch must share device and dtypes"
    options = grad_options(ps[0].device, grad_scale, grad_scale_dev, found_inf, zero_grad, step_consts)
    launch_small_table(arr, ps[0].device, p_tag, g_tag, beta1, beta2, lr, weight_decay, eps, step,
                       options)


def make_salts(salts):
    """ctypes uint32 array of per-tensor noise salts for launch_table_sr."""
    import ctypes
    return (ctypes.c_uint32 * len(salts))(*[int(x) & 0xFFFFFFFF for x in salts])


def launch_table_sr(arr, salts_arr, seed, device, p_tag, g_tag, beta1, beta2, lr, weight_decay, eps,
                    step, options=None):
    L = _lib.load()
    assert salts_arr is None or len(salts_arr) == len(arr), "one salt per tensor"
    with _on(device):
        rc = L.q4adamw_fused_4bit_multi_sr(arr, len(arr), salts_arr, int(seed) & (2 ** 64 - 1), p_tag, g_tag,
                                           beta1, beta2, lr, weight_decay, eps, float(step), options,
                                           _stream(device))
    _lib.check(rc, "fused_4bit_multi_sr")


def fused_4bit_multi_sr(ps, gs, exps, sqs, exp_scales, sq_scales, beta1, beta2, lr, weight_decay, eps,
                        step, seed, salts=None, grad_scale=1.0, grad_scale_dev=None, found_inf=None,
                        zero_grad=False, update_form="auto"):
    """fused_4bit_multi with stochastic rounding of both moments (the rule quoted at
    optim/adamw_fourbit_triton.py:1050-1075).  The noise is a function of (seed, step, the
    tensor's salt, element index): salts defaults to the tensors' positions in the list."""
    if not ps:
        return
    arr = make_table(ps, gs, exps, sqs, exp_scales, sq_scales)
    p_tag, g_tag = _tag(ps[0], "param"), _tag(gs[0], "grad")
    for p, g in zip(ps, gs):
        assert p.device == ps[0].device and _tag(p, "param") == p_tag and _tag(g, "grad") == g_tag, \
            "tensors of one launch must share device and dtypes"
    options = grad_options(ps[0].device, grad_scale, grad_scale_dev, found_inf, zero_grad,
                           update_form=update_form)
    launch_table_sr(arr, None if salts is None else make_salts(salts), seed, ps[0].device, p_tag, g_tag,
                    beta1, beta2, lr, weight_decay, eps, step, options)


def rank1_eligible(p):
    """Whether the second moment of `p` can be rank-1 scaled: every tensor of two to four
    dimensions, as the draft scales every tensor with dim() > 1
    (optim/adamw_fourbit_triton.py:841-846).  Left on block scales, like 1-D tensors there: a
    last dimension of 1 (a column is a vector laid out flat), five and more dimensions, and --
    a limit of the kernel for rows that are no multiple of 8 elements long or shorter than 16
    -- such tensors of 2^32 elements and more."""
    if not 2 <= p.dim() <= 4 or p.shape[-1] < 2:
        return False
    aligned_rows = p.shape[-1] % 8 == 0 and p.shape[-1] >= 16
    return aligned_rows or p.numel() < (1 << 32)


def rank1_row_scale(lead_maxes, lead_shape):
    """Scale of every flattened row of a tensor with several leading dimensions: the minimum
    over the row's leading statistics (compute_variance_tensor_scale without the last
    dimension, optim/adamw_fourbit_triton.py:749-755).  lead_maxes: one float32 tensor per
    leading dimension with lead_shape[j] elements.  Returns a flat float32 tensor."""
    k = len(lead_shape)
    scale = None
    for j, m in enumerate(lead_maxes):
        view = m.reshape([lead_shape[j] if d == j else 1 for d in range(k)])
        scale = view if scale is None else torch.minimum(scale, view)
    return scale.expand(list(lead_shape)).reshape(-1).contiguous()


def check_rank1(p, g, exp, sq, exp_scale, row_max, col_max, row_next, col_next, lead=None):
    _check_common(p, g)
    assert rank1_eligible(p), "rank-1 scaling needs 2 to 4 dimensions, the last of at least 2"
    cols = p.shape[-1]
    rows = p.numel() // cols
    assert (lead is None) == (p.dim() == 2), "tensors of more than two dimensions need their leading statistics"
    if lead is not None:
        lead_maxes, lead_nexts = lead
        assert len(lead_maxes) == len(lead_nexts) == p.dim() - 1, "one statistic per leading dimension"
        for j, (m, nx) in enumerate(zip(lead_maxes, lead_nexts)):
            for t in (m, nx):
                assert t.dtype == torch.float32 and t.numel() == p.shape[j] and t.device == p.device \
                    and t.is_contiguous(), f"leading statistic {j} must be {p.shape[j]} float32 on the param's device"
    nbytes, nblk = state_sizes(p.numel())
    assert exp.dtype == torch.uint8 and sq.dtype == torch.uint8, "moments must be packed uint8"
    assert exp.numel() == nbytes and sq.numel() == nbytes, f"packed moments must hold {nbytes} bytes"
    assert exp_scale.dtype == torch.float32 and exp_scale.numel() == nblk, f"exp_avg scales must hold {nblk} blocks"
    for t, n, what in ((row_max, rows, "row"), (row_next, rows, "row"), (col_max, cols, "column"),
                       (col_next, cols, "column")):
        assert t.dtype == torch.float32 and t.numel() == n, f"{what} maxima must be {n} float32"
    for t in (exp, sq, exp_scale, row_max, col_max, row_next, col_next):
        assert t.device == p.device and t.is_contiguous(), "state must be contiguous on the param's device"


def make_rank1_table(ps, gs, exps, sqs, exp_scales, row_maxes, col_maxes, row_nexts, col_nexts, leads=None):
    """leads: None, or per tensor None (a matrix) or (leading statistics, their scratch), two
    lists with one float32 tensor per leading dimension; row_maxes[i] then holds the flattened
    rows' scales (rank1_row_scale)."""
    n = len(ps)
    arr = (_lib.Q4Rank1Tensor * n)()
    for i in range(n):
        lead = None if leads is None else leads[i]
        check_rank1(ps[i], gs[i], exps[i], sqs[i], exp_scales[i], row_maxes[i], col_maxes[i],
                    row_nexts[i], col_nexts[i], lead)
        a = arr[i]
        a.p, a.g = ps[i].data_ptr(), gs[i].data_ptr()
        a.exp_avg, a.exp_avg_sq = exps[i].data_ptr(), sqs[i].data_ptr()
        a.exp_avg_scale = exp_scales[i].data_ptr()
        a.row_max, a.col_max = row_maxes[i].data_ptr(), col_maxes[i].data_ptr()
        a.row_max_next, a.col_max_next = row_nexts[i].data_ptr(), col_nexts[i].data_ptr()
        a.cols = ps[i].shape[-1]
        a.rows = ps[i].numel() // a.cols
        if lead is not None:
            a.lead_dims = ps[i].dim() - 1
            for j in range(a.lead_dims):
                a.lead_shape[j] = ps[i].shape[j]
                a.lead_max[j] = lead[0][j].data_ptr()
                a.lead_max_next[j] = lead[1][j].data_ptr()
    return arr


def launch_rank1_table(arr, device, p_tag, g_tag, beta1, beta2, lr, weight_decay, eps, step,
                       options=None):
    L = _lib.load()
    with _on(device):
        rc = L.q4adamw_fused_4bit_rank1_multi(arr, len(arr), p_tag, g_tag, beta1, beta2, lr,
                                              weight_decay, eps, float(step), options, _stream(device))
    _lib.check(rc, "fused_4bit_rank1_multi")


def launch_rank1_table_sr(arr, salts_arr, seed, device, p_tag, g_tag, beta1, beta2, lr, weight_decay,
                          eps, step, options=None):
    L = _lib.load()
    assert salts_arr is None or len(salts_arr) == len(arr), "one salt per tensor"
    with _on(device):
        rc = L.q4adamw_fused_4bit_rank1_multi_sr(arr, len(arr), salts_arr, int(seed) & (2 ** 64 - 1), p_tag,
                                                 g_tag, beta1, beta2, lr, weight_decay, eps, float(step),
                                                 options, _stream(device))
    _lib.check(rc, "fused_4bit_rank1_multi_sr")


def fused_4bit_rank1_multi(ps, gs, exps, sqs, exp_scales, row_maxes, col_maxes, row_nexts, col_nexts,
                           beta1, beta2, lr, weight_decay, eps, step, grad_scale=1.0,
                           grad_scale_dev=None, found_inf=None, zero_grad=False, seed=None, salts=None,
                           step_consts=None, leads=None, update_form="auto"):
    """The fused step over matrices whose second moment is rank-1 scaled: scale of element
    (i, j) = min(row_maxes[i], col_maxes[j]).  row_nexts / col_nexts are state-owned scratch
    that holds zeros between steps.  Gradient options as for fused_4bit_multi.  With a seed
    both moments are rounded stochastically, noise and salts as for fused_4bit_multi_sr."""
    if not ps:
        return
    arr = make_rank1_table(ps, gs, exps, sqs, exp_scales, row_maxes, col_maxes, row_nexts, col_nexts, leads)
    p_tag, g_tag = _tag(ps[0], "param"), _tag(gs[0], "grad")
    for p, g in zip(ps, gs):
        assert p.device == ps[0].device and _tag(p, "param") == p_tag and _tag(g, "grad") == g_tag, \
            "tensors of one launch must share device and dtypes"
    options = grad_options(ps[0].device, grad_scale, grad_scale_dev, found_inf, zero_grad, step_consts,
                           update_form)
    if seed is None:
        launch_rank1_table(arr, ps[0].device, p_tag, g_tag, beta1, beta2, lr, weight_decay, eps, step, options)
    else:
        launch_rank1_table_sr(arr, None if salts is None else make_salts(salts), seed, ps[0].device, p_tag,
                              g_tag, beta1, beta2, lr, weight_decay, eps, step, options)


def make_grad_table(gs):
    """ctypes descriptor array for grad_norm_table (gradients validated)."""
    arr = (_lib.Q4Grad * len(gs))()
    for i, g in enumerate(gs):
        assert g.is_cuda and g.device == gs[0].device, "gradients must share a cuda device"
        assert g.is_contiguous(), "grad must be contiguous"
        assert g.dtype == gs[0].dtype, "gradients of one call must share a dtype"
        arr[i].g, arr[i].numel = g.data_ptr(), g.numel()
    return arr


def grad_norm_table(arr, device, g_tag, out3, workspace, grad_scale=1.0, grad_scale_dev=None,
                    max_norm=0.0):
    L = _lib.load()
    assert out3.dtype == torch.float32 and out3.numel() >= 3 and out3.device == device
    assert workspace.device == device and workspace.numel() * workspace.element_size() >= _lib.NORM_WORKSPACE_BYTES
    dev_ptr = None if grad_scale_dev is None else _device_scalar(grad_scale_dev, device, "grad_scale_dev")
    with torch.cuda.device(device):
        rc = L.q4adamw_grad_norm(arr, len(arr), g_tag, float(grad_scale), dev_ptr, float(max_norm),
                                 workspace.data_ptr(), workspace.numel() * workspace.element_size(),
                                 out3.data_ptr(), _stream(device))
    _lib.check(rc, "grad_norm")


def grad_norm(gs, grad_scale=1.0, grad_scale_dev=None, max_norm=0.0, out=None, workspace=None):
    """Global L2 norm of the gradients `gs` (one dtype, one device) and the clip coefficient of
    torch.nn.utils.clip_grad_norm_.  Returns a device float32[3]: the norm of the gradients
    times s = grad_scale * grad_scale_dev, min(1, max_norm / (norm + 1e-6)) (1 when max_norm
    <= 0), and s times that coefficient -- the multiplier to pass to a step as
    grad_scale_dev.  Nothing is synchronised."""
    assert len(gs) > 0, "no gradients"
    device = gs[0].device
    if out is None:
        out = torch.empty(3, dtype=torch.float32, device=device)
    if workspace is None:
        workspace = torch.empty(_lib.NORM_WORKSPACE_BYTES // 8, dtype=torch.float64, device=device)
    grad_norm_table(make_grad_table(gs), device, _tag(gs[0], "grad"), out, workspace, grad_scale,
                    grad_scale_dev, max_norm)
    return out


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


def quantize_state_rank1(x):
    """fp32 second moment of a matrix (on a GPU) -> (packed uint8 codes, row maxima [rows],
    column maxima [cols]); element (i, j) is divided by min(row_max[i], col_max[j]).  Device
    form of variance_quant with rank-1 scaling (optim/adamw_fourbit_triton.py:803-863)."""
    L = _lib.load()
    assert x.is_cuda and x.dim() == 2, "needs a cuda matrix"
    x = x.detach().to(torch.float32).contiguous()
    rows, cols = x.shape
    codes = torch.empty((rows * cols + 1) // 2, dtype=torch.uint8, device=x.device)
    row_max = torch.empty(rows, dtype=torch.float32, device=x.device)
    col_max = torch.empty(cols, dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        rc = L.q4adamw_quantize_rank1(x.data_ptr(), rows, cols, codes.data_ptr(), row_max.data_ptr(),
                                      col_max.data_ptr(), _stream(x.device))
    _lib.check(rc, "quantize_rank1")
    return codes, row_max, col_max


def quantize_state_rank1_scaled(x, row_scale, col_max):
    """fp32 second moment viewed as a matrix [rows, cols] -> packed codes, every element divided
    by min(row_scale[i], col_max[j]): the quantizer for tensors of more than two dimensions,
    whose rows' scales come from rank1_row_scale."""
    L = _lib.load()
    assert x.is_cuda and x.dim() == 2, "needs a cuda matrix"
    x = x.detach().to(torch.float32).contiguous()
    rows, cols = x.shape
    for t, n in ((row_scale, rows), (col_max, cols)):
        assert t.dtype == torch.float32 and t.numel() == n and t.device == x.device and t.is_contiguous()
    codes = torch.empty((rows * cols + 1) // 2, dtype=torch.uint8, device=x.device)
    with torch.cuda.device(x.device):
        rc = L.q4adamw_quantize_rank1_scaled(x.data_ptr(), rows, cols, row_scale.data_ptr(), col_max.data_ptr(),
                                             codes.data_ptr(), _stream(x.device))
    _lib.check(rc, "quantize_rank1_scaled")
    return codes


def dequantize_state_rank1(codes, row_max, col_max):
    """(packed codes, row maxima, column maxima) -> fp32 matrix [rows, cols]
    (optim/adamw_fourbit_triton.py:520-527)."""
    L = _lib.load()
    rows, cols = row_max.numel(), col_max.numel()
    assert codes.is_cuda and codes.dtype == torch.uint8 and codes.numel() == (rows * cols + 1) // 2
    for t in (row_max, col_max):
        assert t.dtype == torch.float32 and t.device == codes.device and t.is_contiguous()
    out = torch.empty(rows, cols, dtype=torch.float32, device=codes.device)
    with torch.cuda.device(codes.device):
        rc = L.q4adamw_dequantize_rank1(codes.data_ptr(), row_max.data_ptr(), col_max.data_ptr(), rows, cols,
                                        out.data_ptr(), _stream(codes.device))
    _lib.check(rc, "dequantize_rank1")
    return out


def rounding_selfcheck(device):
    """q4adamw_rounding_selfcheck on `device`: dict of the six counters (sqrt, reciprocal,
    quotient, general_sqrt, general_quotient mismatches -- all must be 0 -- and walked)."""
    L = _lib.load()
    counts = torch.zeros(6, dtype=torch.int64, device=device)
    with _on(device):
        rc = L.q4adamw_rounding_selfcheck(counts.data_ptr(), _stream(device))
    _lib.check(rc, "rounding_selfcheck")
    names = ("sqrt", "reciprocal", "quotient", "general_sqrt", "general_quotient", "walked")
    return dict(zip(names, (int(x) for x in counts.cpu())))
