"""The gradient norm without a caller-provided workspace (q4adamw_grad_norm_static), through
the C ABI: its three outputs must equal q4adamw_grad_norm's bit for bit -- both run the same
kernels in the same fixed summation order, only the home of the partial sums differs (a
16 KiB array inside the library's device image instead of device memory the caller brings).

Two calls in a row, the second on a smaller input: the array keeps the first call's partial
sums, and the second call must not see them.  Collected last (the file's name sorts after
the other test files), and it passes alone in a fresh process as well as after the others.
"""

import numpy as np
import pytest
import torch

from oracle import q4_oracle as oc
from quantfour_adamw_cuda_amd import _lib
from tests.q4_testlib import to_np

pytestmark = pytest.mark.gpu

DT = {"fp32": (torch.float32, _lib.FP32), "bf16": (torch.bfloat16, _lib.BF16), "fp16": (torch.float16, _lib.FP16)}


def _table(gs):
    arr = (_lib.Q4Grad * len(gs))()
    for i, g in enumerate(gs):
        arr[i].g, arr[i].numel = g.data_ptr(), g.numel()
    return arr


def _both(L, gs, tag, scale, scale_dev, max_norm, device, poison=False):
    """(static entry point's out3, workspace entry point's out3) as uint32 bit patterns"""
    stream = torch.cuda.current_stream(device).cuda_stream
    arr = _table(gs)
    sd = None if scale_dev is None else scale_dev.data_ptr()
    out_static = torch.full((3,), -7.0, dtype=torch.float32, device=device)
    out_ws = torch.full((3,), -9.0, dtype=torch.float32, device=device)
    ws = torch.empty(_lib.NORM_WORKSPACE_BYTES // 8, dtype=torch.float64, device=device)
    if poison:
        ws.fill_(float("nan"))
    rc = L.q4adamw_grad_norm_static(arr, len(gs), tag, scale, sd, max_norm, out_static.data_ptr(), stream)
    assert rc == 0, L.q4adamw_last_error()
    rc = L.q4adamw_grad_norm(arr, len(gs), tag, scale, sd, max_norm, ws.data_ptr(),
                             ws.numel() * 8, out_ws.data_ptr(), stream)
    assert rc == 0, L.q4adamw_last_error()
    torch.cuda.synchronize(device)
    return out_static.cpu().numpy().view(np.uint32), out_ws.cpu().numpy().view(np.uint32)


@pytest.mark.parametrize("g_dt", ["bf16", "fp32", "fp16"])
def test_static_scratch_matches_workspace_two_calls(cuda, g_dt):
    L = _lib.load()
    dtype, tag = DT[g_dt]
    gen = torch.Generator().manual_seed(31)
    # first call: several tensors, more chunks than workgroups (every partial sum is used),
    # ragged tails; second call: one small tensor, so most partial sums must read as zero
    big = [(torch.randn(n, generator=gen) * 3.0).to(dtype).to(cuda) for n in (5_000_011, 16384 * 300, 129, 1)]
    small = [(torch.randn(777, generator=gen) * 0.01).to(dtype).to(cuda)]
    scale_dev = torch.tensor([0.25], device=cuda)
    a_static, a_ws = _both(L, big, tag, 0.5, scale_dev, 1.0, cuda)
    assert np.array_equal(a_static, a_ws), f"first call: {a_static} vs {a_ws}"
    b_static, b_ws = _both(L, small, tag, 1.0, None, 1e-3, cuda, poison=True)
    assert np.array_equal(b_static, b_ws), f"second, smaller call: {b_static} vs {b_ws}"
    # and both agree with the CPU oracle's norm (fp64 sum of exact squares), so that equality
    # above is not two wrong answers: norm within fp32 round-off of the oracle's
    norm, coef, mult = oc.grad_norm([to_np(g) for g in small], np.float32(1.0), 1e-3)
    got = b_static.view(np.float32)
    assert abs(got[0] - norm) <= 2e-7 * norm and abs(got[1] - coef) <= 4e-7 * coef and abs(got[2] - mult) <= 4e-7 * abs(mult)
    # an empty list: norm 0, coefficient 1 -- nothing left over from the calls before
    e_static, e_ws = _both(L, [torch.zeros(0, dtype=dtype, device=cuda)], tag, 1.0, None, 1.0, cuda)
    assert np.array_equal(e_static, e_ws) and e_static.view(np.float32)[0] == 0.0 and e_static.view(np.float32)[1] == 1.0


def test_static_scratch_refusals(cuda):
    """the argument checks of q4adamw_grad_norm hold here too; nothing is launched on a refusal"""
    L = _lib.load()
    g = torch.ones(64, device=cuda)
    out = torch.zeros(3, device=cuda)
    arr = _table([g])
    call = lambda a, cnt, tag, o: L.q4adamw_grad_norm_static(a, cnt, tag, 1.0, None, 0.0, o, None)
    assert call(arr, 1, _lib.FP32, None) == -1 and b"null" in L.q4adamw_last_error()
    assert call(arr, -1, _lib.FP32, out.data_ptr()) == -1
    assert call(arr, 1, 7, out.data_ptr()) == -1
    arr[0].g = g.data_ptr() + 2
    assert call(arr, 1, _lib.FP32, out.data_ptr()) == -2 and b"element size" in L.q4adamw_last_error()
    arr[0].g, arr[0].numel = g.data_ptr(), 1 << 62
    assert call(arr, 1, _lib.FP32, out.data_ptr()) == -4 and b"too large" in L.q4adamw_last_error()
    torch.cuda.synchronize(cuda)
    assert torch.equal(out.cpu(), torch.zeros(3))


def test_static_scratch_under_graph_capture(cuda):
    """One of the callers the entry point is for: code under graph capture.  The call is recorded
    once (after a first call outside the capture, which is when the library asks the runtime for
    its array's address) and replayed with new gradient values, with the program's own eager
    work between the replays; every replay must give the eager workspace form's bits."""
    L = _lib.load()
    gen = torch.Generator().manual_seed(37)
    gs = [torch.zeros(n, dtype=torch.bfloat16, device=cuda) for n in (3_000_017, 16384 * 40, 5)]
    arr = _table(gs)
    out = torch.zeros(3, device=cuda)

    def fill():
        for g in gs:
            g.copy_((torch.randn(g.numel(), generator=gen) * 2.0).to(torch.bfloat16))

    fill()
    side = torch.cuda.Stream(device=cuda)
    with torch.cuda.stream(side):
        rc = L.q4adamw_grad_norm_static(arr, len(gs), _lib.BF16, 0.5, None, 1.0, out.data_ptr(), side.cuda_stream)
        assert rc == 0, L.q4adamw_last_error()
    torch.cuda.synchronize(cuda)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        rc = L.q4adamw_grad_norm_static(arr, len(gs), _lib.BF16, 0.5, None, 1.0, out.data_ptr(),
                                        torch.cuda.current_stream(cuda).cuda_stream)
        assert rc == 0, L.q4adamw_last_error()
    for replay in range(4):
        fill()
        _, eager = _both(L, gs, _lib.BF16, 0.5, None, 1.0, cuda, poison=True)   # eager work in between
        out.fill_(-1.0)
        graph.replay()
        torch.cuda.synchronize(cuda)
        got = out.cpu().numpy().view(np.uint32)
        assert np.array_equal(got, eager), f"replay {replay}: {got} vs {eager}"
